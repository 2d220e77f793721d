"""GPU parity of adaptive block-sparse attention vs the CPU oracle.  Mask estimate: the reference's own
tolerance for its kernel against the numpy statement (tests/plugin/test_sparseblockestimate.py:231-241):
differing blocks below 2 % of the selected ones, omitted blocks below 1 %.  Attention: the reference's
kernel rule |err| <= 2^-6 * max(1, |golden|) (tests/plugin/test_adablocksparseattention.py:26-32, :173)."""
import numpy as np
import pytest
import torch

from oracle import ada_bsa as oab
from oracle.attention import ref_compare

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.float16, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * mul).to(dtype)


def _structured(shape, seed, dtype):
    """Scores with structure: a slowly varying component shared by neighbouring tokens plus noise."""
    b, n, s, d = shape
    base = _rand((b, n, (s + 63) // 64, d), seed, torch.float32).repeat_interleave(64, dim=2)[:, :, :s]
    return (base + 0.5 * _rand(shape, seed + 1, torch.float32)).to(dtype)


def _mask_close(got, want):
    """The reference's tolerance for its kernel against its numpy statement (test_sparseblockestimate.py:231-241)."""
    selected = want.sum()
    assert (got != want).sum() / selected < 0.02, ((got != want).sum(), selected)
    assert (got < want).sum() / selected < 0.01, ((got < want).sum(), selected)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("s,threshold,row_sparse", [(2048, 0.85, 1.0), (3000, 0.6, 0.5), (1031, 0.9, 1.0)])
def test_sparse_block_estimate_vs_oracle(cuda, s, threshold, row_sparse, dtype):
    import mindiesd  # noqa: F401
    q, k = _structured((1, 2, s, 128), 1, dtype), _structured((1, 2, s, 128), 3, dtype)
    scale = 128 ** -0.5 / 8
    smask, sct = torch.ops.mindiesd.sparse_block_estimate(
        q.to(cuda), k.to(cuda), input_layout="BNSD", stride=8, sparse_size=128, num_heads=2, num_key_value_heads=2,
        scale_value=scale, threshold=threshold, causal=False, keep_sink=True, keep_recent=True, row_sparse=row_sparse)
    nb = (s + 127) // 128
    assert smask.shape == (1, 2, nb, (nb + 31) // 32 * 32) and smask.dtype == torch.int8
    assert sct.shape == (1, 2, nb) and sct.dtype == torch.int32
    got = smask.cpu().numpy().astype(bool)
    assert not got[..., nb:].any()
    assert np.array_equal(sct.cpu().numpy(), got.sum(-1))
    want = oab.sparse_estimate(q, k, threshold=threshold, force_sparse=row_sparse, rules="kernel")
    got = got[..., :nb]
    assert got[..., 0].all() and got[..., -1].all()
    for h in range(2):
        _mask_close(got[0, h], want[0, h])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sign", [-1.0, 1.0, 0.0])
def test_estimate_on_scores_far_from_zero(cuda, sign, dtype):
    """q near +8 and k near -8 / +8 (every strided score hundreds of units below / above zero), and all-zero inputs
    (uniform rows): the running maxima of the score kernel start from nothing in every case."""
    import mindiesd  # noqa: F401
    g = torch.Generator().manual_seed(5)
    q = ((8.0 + 0.5 * torch.randn((1, 2, 2048, 128), generator=g)) * abs(sign)).to(dtype)
    k = ((8.0 * sign + 0.5 * torch.randn((1, 2, 2048, 128), generator=g)) * abs(sign)).to(dtype)
    smask, sct = torch.ops.mindiesd.sparse_block_estimate(
        q.to(cuda), k.to(cuda), input_layout="BNSD", stride=8, sparse_size=128, num_heads=2, num_key_value_heads=2,
        scale_value=128 ** -0.5 / 8, threshold=0.85, causal=False, keep_sink=True, keep_recent=True, row_sparse=1.0)
    got = smask.cpu().numpy().astype(bool)
    assert np.array_equal(sct.cpu().numpy(), got.sum(-1))
    want = oab.sparse_estimate(q, k, threshold=0.85, force_sparse=1.0, rules="kernel")
    for h in range(2):
        _mask_close(got[0, h, :, :16], want[0, h])


def test_estimate_against_the_numpy_statement_on_the_reference_test_case(cuda):
    """The reference's own test (tests/plugin/test_sparseblockestimate.py:150-241): B1 N1 S8192 D128, N(0,1) inputs
    cast to fp16, threshold 0.85, no cap, default switches, kernel against the numpy statement within 2 % / 1 %."""
    import mindiesd  # noqa: F401
    q, k = _rand((1, 1, 8192, 128), 0), _rand((1, 1, 8192, 128), 1)
    smask, sct = torch.ops.mindiesd.sparse_block_estimate(
        q.to(cuda), k.to(cuda), input_layout="BNSD", stride=8, sparse_size=128, num_heads=1, num_key_value_heads=1,
        scale_value=128 ** -0.5 / 8, threshold=0.85, causal=False, keep_sink=True, keep_recent=True, row_sparse=1.0)
    assert smask.shape == (1, 1, 64, 64) and sct.shape == (1, 1, 64)
    want = oab.sparse_estimate(q, k, threshold=0.85, force_sparse=1.0, rules="numpy")
    _mask_close(smask.cpu().numpy().astype(bool)[0, 0], want[0, 0])


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
def test_block_scores_layouts_heads_and_workspace_groups(cuda, layout):
    """Scores of the fused kernel against the oracle's block scores: grouped-query heads, both layouts, a batch,
    a sequence that is no multiple of 8, and a workspace that only holds two of the six heads at a time."""
    from mindiesd import _native
    s, b, n, nkv = 2707, 2, 3, 1
    q, k = _structured((b, n, s, 128), 31, torch.bfloat16), _structured((b, nkv, s, 128), 33, torch.bfloat16)
    qd, kd = (t.to(cuda) if layout == "BNSD" else t.transpose(1, 2).contiguous().to(cuda).transpose(1, 2) for t in (q, k))
    nb = (s + 127) // 128
    lib = _native.lib()
    scores = torch.full((b * n, nb, nb), -1.0, dtype=torch.float32, device=cuda)
    ws_bytes = lib.mindiesd_sbe_scores_workspace_size(2, s)
    assert ws_bytes * 3 == lib.mindiesd_sbe_scores_workspace_size(6, s)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    rc = lib.mindiesd_sbe_scores(qd.data_ptr(), kd.data_ptr(), scores.data_ptr(), 0, b, n, nkv, s, 128,
                                 qd.stride(0), qd.stride(1), qd.stride(2), kd.stride(0), kd.stride(1), kd.stride(2),
                                 128 ** -0.5 / 8, 0, ws.data_ptr(), ws_bytes, _native.stream_ptr(cuda))
    assert rc == 0
    got = scores.cpu().numpy().reshape(b, n, nb, nb)
    for bi in range(b):
        for ni in range(n):
            want = oab.block_scores(q[bi, ni].float().numpy(), k[bi, 0].float().numpy())
            assert np.abs(got[bi, ni] - want).max() < 2e-3, (bi, ni, np.abs(got[bi, ni] - want).max())
            assert abs(got[bi, ni].sum() - (s + 7) // 8) < 0.05
    # too small a workspace and bad arguments are refused
    assert lib.mindiesd_sbe_scores(qd.data_ptr(), kd.data_ptr(), scores.data_ptr(), 0, b, n, nkv, s, 128,
                                   qd.stride(0), qd.stride(1), qd.stride(2), kd.stride(0), kd.stride(1), kd.stride(2),
                                   0.01, 0, ws.data_ptr(), ws_bytes // 2 - 16, _native.stream_ptr(cuda)) == 3
    assert lib.mindiesd_sbe_scores(qd.data_ptr(), kd.data_ptr(), scores.data_ptr(), 0, b, n, nkv, s, 64,
                                   qd.stride(0), qd.stride(1), qd.stride(2), kd.stride(0), kd.stride(1), kd.stride(2),
                                   0.01, 0, ws.data_ptr(), ws_bytes, _native.stream_ptr(cuda)) == 2


@pytest.mark.parametrize("keep_recent", [True, False])
@pytest.mark.parametrize("s,threshold,row_sparse", [(2048, 0.85, 1.0), (3000, 0.6, 0.5), (1031, 0.9, 1.0)])
def test_causal_sparse_block_estimate_vs_oracle(cuda, s, threshold, row_sparse, keep_recent):
    """Causal estimate: keys limited per step of 1024 query tokens, selection inside the lower triangle."""
    import mindiesd  # noqa: F401
    from mindiesd.layers.flash_attn.ada_bsa import sparse_block_estimate
    q, k = _structured((1, 2, s, 128), 11, torch.float16), _structured((1, 2, s, 128), 13, torch.float16)
    scale = 128 ** -0.5 / 8
    smask, sct, scores = sparse_block_estimate(q.to(cuda), k.to(cuda), scale_value=scale, threshold=threshold,
                                               causal=True, keep_recent=keep_recent, row_sparse=row_sparse,
                                               return_scores=True)
    nb = (s + 127) // 128
    got = smask.cpu().numpy().astype(bool)[..., :nb]
    assert np.array_equal(sct.cpu().numpy(), got.sum(-1))
    assert not np.triu(got[0, 0], 1).any() and not np.triu(got[0, 1], 1).any()
    assert got[0, :, 0, 0].all() and got[0, :, 1, :2].all()
    want_sc = oab.block_scores(q[0, 0].float().numpy(), k[0, 0].float().numpy(), causal=True)
    got_sc = scores.cpu().numpy()[0, 0]
    assert np.abs(got_sc[:, :want_sc.shape[1]] - want_sc[:nb, :nb]).max() < 2e-3
    want = oab.sparse_estimate(q, k, threshold=threshold, force_sparse=row_sparse, keep_recent=keep_recent,
                               causal=True, rules="kernel")
    for h in range(2):
        _mask_close(got[0, h], want[0, h])
    if keep_recent:
        assert np.diag(got[0, 0]).all()


@pytest.mark.parametrize("keep_sink,keep_recent", [(True, True), (False, True), (True, False), (False, False)])
def test_block_scores_and_selection_separately(cuda, keep_sink, keep_recent):
    from mindiesd.layers.flash_attn.ada_bsa import sparse_block_estimate
    s = 2500
    q, k = _structured((1, 1, s, 128), 5, torch.float16), _structured((1, 1, s, 128), 7, torch.float16)
    mask, cnt, scores = sparse_block_estimate(q.to(cuda), k.to(cuda), scale_value=128 ** -0.5 / 8, threshold=0.8,
                                              row_sparse=0.7, keep_sink=keep_sink, keep_recent=keep_recent,
                                              return_scores=True)
    want = oab.block_scores(q[0, 0].float().numpy(), k[0, 0].float().numpy())
    got = scores.cpu().numpy()[0, 0]
    nb = (s + 127) // 128
    assert got.shape == (nb, nb)
    # exact 16-bit inputs, fp32 accumulation: block masses agree to a small fraction of a row's mass (16)
    assert np.abs(got - want).max() < 2e-3 and abs(got.sum() - (s + 7) // 8) < 0.05
    # the selection kernel on the GPU's own scores reproduces the kernel rules row by row
    sel = np.stack([oab.select_blocks_kernel(got[i], 0.8, 0.7, keep_sink, keep_recent) for i in range(nb)])
    assert (mask.cpu().numpy()[0, 0, :, :nb].astype(bool) != sel).mean() < 1e-3
    assert np.array_equal(cnt.cpu().numpy()[0, 0], mask.cpu().numpy()[0, 0].sum(-1))


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("causal", [False, True])
def test_ada_block_sparse_attention_vs_oracle(cuda, causal, layout):
    import mindiesd  # noqa: F401
    s, nb = 1100, 9
    q, k, v = _rand((1, 4, s, 128), 9, torch.bfloat16), _rand((1, 2, s, 128), 10, torch.bfloat16), _rand((1, 2, s, 128), 11, torch.bfloat16)
    g = torch.Generator().manual_seed(12)
    m = torch.rand(1, 4, nb, nb, generator=g) > 0.5
    m[:, :, torch.arange(nb), torch.arange(nb)] = True
    if causal:
        m &= torch.ones(nb, nb).tril().bool()
    m[0, 3, 4] = False if not causal else m[0, 3, 4]
    smask = torch.zeros(1, 4, nb, 32, dtype=torch.int8)
    smask[..., :nb] = m.to(torch.int8)
    sct = m.sum(-1).to(torch.int32)
    want = oab.ada_block_sparse_attention(q, k, v, m.numpy(), causal=causal)
    args = (q, k, v) if layout == "BNSD" else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = torch.ops.mindiesd.ada_block_sparse_attention(
        *(t.to(cuda) for t in args), smask.to(cuda), sct.to(cuda), input_layout=layout, sparse_size=128, num_heads=4,
        num_key_value_heads=2, scale_value=128 ** -0.5, causal=causal).cpu()
    out = out if layout == "BNSD" else out.transpose(1, 2)
    eb, ok, mx = ref_compare(want, out, 2.0 ** -6)
    assert ok, (eb, mx)
    if not causal:
        assert not out[0, 3, 512:640].any()


@pytest.mark.parametrize("seed", range(6))
def test_ada_attention_causal_rows_without_their_diagonal_block(cuda, seed):
    """Random masks inside the lower triangle whose rows need not end with their diagonal block.  The reference
    kernel masks inside a block only when the row's last selected block is the diagonal one
    (ada_block_sparse_attention_s1s2_bns1_x910.h:512-514); its numpy test statement masks the last selected block
    whatever it is.  The build tests key <= query by token index, which is the kernel's rule on such masks."""
    import mindiesd  # noqa: F401
    g = torch.Generator().manual_seed(seed)
    s = (500, 769, 1100, 1537, 256, 130)[seed]
    nb = (s + 127) // 128
    q, k, v = _rand((2, 4, s, 128), seed, torch.bfloat16), _rand((2, 2, s, 128), seed + 1, torch.bfloat16), _rand((2, 2, s, 128), seed + 2, torch.bfloat16)
    m = (torch.rand(2, 4, nb, nb, generator=g) > 0.5) & torch.ones(nb, nb).tril().bool()
    smask = torch.zeros(2, 4, nb, 32, dtype=torch.int8)
    smask[..., :nb] = m.to(torch.int8)
    want = oab.ada_block_sparse_attention(q, k, v, m.numpy(), causal=True, rules="kernel")
    out = torch.ops.mindiesd.ada_block_sparse_attention(
        q.to(cuda), k.to(cuda), v.to(cuda), smask.to(cuda), m.sum(-1).to(torch.int32).to(cuda), input_layout="BNSD",
        sparse_size=128, num_heads=4, num_key_value_heads=2, scale_value=128 ** -0.5, causal=True).cpu()
    eb, ok, mx = ref_compare(want, out, 2.0 ** -6)
    assert ok, (eb, mx)


def test_sparse_attention_front_door_ada_bsa(cuda):
    from mindiesd import sparse_attention
    from mindiesd.layers.flash_attn.sparse_flash_attn_ada_bsa import get_estimate_mask
    s = 2100
    q, k = _structured((1, 2, s, 128), 13, torch.bfloat16), _structured((1, 2, s, 128), 15, torch.bfloat16)
    v = _rand((1, 2, s, 128), 17, torch.bfloat16)
    out = sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), head_num=2, input_layout="BNSD", sparse_type="ada_bsa",
                           cdf_threshold=0.8, sparsity=0.3).cpu()
    smask, _ = get_estimate_mask(q.to(cuda), k.to(cuda), v.to(cuda), scale=128 ** -0.5, head_num=2, cdf_threshold=0.8,
                                 sparsity=0.3)
    nb = (s + 127) // 128
    want = oab.ada_block_sparse_attention(q, k, v, smask.cpu().numpy()[..., :nb].astype(bool))
    assert ref_compare(want, out, 2.0 ** -6)[1]
    density = smask.float().sum() / (2 * nb * nb)
    assert 0.05 < density <= 0.75


@pytest.mark.parametrize("shape,check_heads", [((1, 12, 32760, 128), (0, 11)), ((1, 40, 75600, 128), (39,))])
def test_sparse_block_estimate_long_sequences(cuda, shape, check_heads):
    """The two DiT shapes (Wan2.1-1.3B and 14B 720p): block scores of the checked heads against the oracle, unit mass
    per strided row in every head, masks of the checked heads within the reference's tolerance."""
    from mindiesd.layers.flash_attn import ada_bsa
    b, n, s, d = shape
    q = torch.cat([_structured((1, 1, s, d), 21 + 2 * h, torch.bfloat16) for h in range(n)], dim=1)
    k = torch.cat([_structured((1, 1, s, d), 121 + 2 * h, torch.bfloat16) for h in range(n)], dim=1)
    print(f"estimate at {shape}", flush=True)
    mask, cnt, scores = ada_bsa.sparse_block_estimate(q.to(cuda), k.to(cuda), scale_value=d ** -0.5 / 8, threshold=0.9,
                                                      row_sparse=0.25, return_scores=True)
    nb = (s + 127) // 128
    assert mask.shape == (1, n, nb, (nb + 31) // 32 * 32) and int(cnt.min()) >= 2
    sc = scores.cpu().numpy()[0]
    rows = np.full(nb, 16.0)
    rows[-1] = (s + 7) // 8 - 16 * (nb - 1)
    assert np.abs(sc.sum(-1) - rows).max() < 1e-2          # every strided row carries probability mass 1
    got = mask.cpu().numpy().astype(bool)[0, :, :, :nb]
    assert np.array_equal(cnt.cpu().numpy()[0], got.sum(-1))
    for h in check_heads:
        want_sc = oab.block_scores(q[0, h].float().numpy(), k[0, h].float().numpy())
        assert np.abs(sc[h] - want_sc).max() < 2e-3, (h, np.abs(sc[h] - want_sc).max())
        want = np.stack([oab.select_blocks_kernel(want_sc[i], 0.9, 0.25) for i in range(nb)])
        _mask_close(got[h], want)


def test_ada_bsa_errors(cuda):
    import mindiesd  # noqa: F401
    q = torch.randn(1, 1, 256, 128, dtype=torch.float16, device=cuda)
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.sparse_block_estimate(q, q, input_layout="TND", causal=False)
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.sparse_block_estimate(q, q, stride=4, causal=False)
    m = torch.ones(1, 1, 2, 32, dtype=torch.int8, device=cuda)
    c = torch.full((1, 1, 2), 2, dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.ada_block_sparse_attention(q, q, q, m[:, :, :1], c, causal=False)
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.ada_block_sparse_attention(q, q, q, m, c, sparse_size=64, causal=False)
