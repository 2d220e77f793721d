"""GPU parity of the RainFusion2.0 pipeline vs the CPU oracle: permutation, pooling and block masks
bit-exact; block-sparse attention within the reference's kernel tolerance
(|err| <= 2^-6 * max(1, |golden|), tests/plugin/test_adablocksparseattention.py:26-32,173)."""
import math

import pytest
import torch

from oracle import rainfusion as orf
from oracle.attention import attention_math, block_sparse_attention, ref_compare

pytestmark = pytest.mark.gpu

# grids of the reference's own tests (tests/layers/flash_attn/test_sparse_flash_attn_rf_v2.py:32-38)
GRIDS = {"div": (3, 40, 80), "nodiv_both": (3, 30, 52), "nodiv_h": (2, 21, 32), "nodiv_w": (2, 24, 45)}


def _rand(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


def _shape(layout, b, n, s, d=128):
    return (b, n, s, d) if layout == "BNSD" else (b, s, n, d)


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid", list(GRIDS))
def test_rearrange_bit_exact_and_round_trip(cuda, grid, layout):
    from mindiesd.layers.flash_attn import rainfusion as rf
    t, h, w = GRIDS[grid]
    x = _rand(_shape(layout, 1, 2, t * h * w), seed=1)
    got = rf.rearrange_with_remaining(x.to(cuda), (t, h, w), (t, h, w), layout)
    assert torch.equal(got.cpu(), orf.rearrange_with_remaining(x, (t, h, w), None, layout))
    back = rf.inv_rearrange_with_remaining(got, (t, h, w), (t, h, w), layout)
    assert torch.equal(back.cpu(), x)
    # the rf_v3 spelling of the inverse (rf_v3.py:22-97)
    from mindiesd.layers.flash_attn.sparse_flash_attn_rf_v3 import _bsa_inv_rearrange
    assert torch.equal(_bsa_inv_rearrange(got, t, h, w, layout).cpu(), x)


def test_do_tensor_pooling_as_the_reference_writes_it(cuda):
    """rf_v2.py:340-348: cut along dim 1, pool both parts along dim 2 (avgpool's default layout), join along dim 1."""
    from mindiesd.layers.flash_attn.sparse_flash_attn_rf_v2 import do_tensor_pooling
    x = _rand((2, 5, 300, 128), seed=4)
    got = do_tensor_pooling(x.to(cuda), 2).cpu()
    want = torch.cat([orf.avgpool(x[:, :2], 128, "BNSD"), orf.avgpool(x[:, 2:], 128, "BNSD")], dim=1)
    assert got.shape == (2, 5, 3, 128) and torch.equal(got, want)
    assert torch.equal(do_tensor_pooling(x.to(cuda), 0).cpu(), orf.avgpool(x, 128, "BNSD"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("s", [64, 768, 800, 4107])
def test_avgpool_bit_exact(cuda, s, layout, dtype):
    from mindiesd.layers.flash_attn import rainfusion as rf
    x = _rand(_shape(layout, 2, 3, s), seed=s, dtype=dtype)
    got = rf.avgpool(x.to(cuda), 128, layout).cpu()
    want = orf.avgpool(x, 128, layout)
    assert got.shape == want.shape
    assert torch.equal(got, want)


def test_avgpool_known_answer(cuda):
    """Reference KAT (test_sparse_flash_attn_rf_v2.py:104-119): arange(256) -> block means 63.5 / 191.5."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    x = torch.arange(256, dtype=torch.float32).reshape(1, 1, 256, 1).expand(1, 1, 256, 128).to(torch.float16)
    got = rf.avgpool(x.contiguous().to(cuda), 128, "BNSD").float().cpu()
    # fp16 holds 0..255 and both means exactly
    assert got[0, 0, 0, 0].item() == 63.5 and got[0, 0, 1, 0].item() == 191.5
    # in bf16 (8 significant bits) 191.5 is a tie between 191 and 192 and rounds to even
    gb = rf.avgpool(x.to(torch.bfloat16).contiguous().to(cuda), 128, "BNSD").float().cpu()
    assert gb[0, 0, 0, 0].item() == 63.5 and gb[0, 0, 1, 0].item() == 192.0


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid,txt", [("div", 0), ("nodiv_both", 0), ("nodiv_h", 300), ("nodiv_w", 128)])
def test_rearrange_pooling_with_text(cuda, grid, txt, layout):
    from mindiesd.layers.flash_attn import rainfusion as rf
    t, h, w = GRIDS[grid]
    s = t * h * w + txt
    q, k, v = (_rand(_shape(layout, 1, 2, s), seed=i) for i in (1, 2, 3))
    gq, gk, gv, gp = rf.do_tensor_rearrange_pooling(q.to(cuda), k.to(cuda), v.to(cuda), txt, 128, (t, h, w), (t, h, w),
                                                    layout)
    oq, ok, ov, op = orf.do_tensor_rearrange_pooling(q, k, v, txt, 128, (t, h, w), (t, h, w), layout)
    for a, b in ((gq, oq), (gk, ok), (gv, ov), (gp, op)):
        assert a.shape == b.shape
        assert torch.equal(a.cpu(), b)
    back = rf.do_tensor_inv_rearrange(gq, txt, (t, h, w), (t, h, w), layout)
    assert torch.equal(back.cpu(), q)


def _structured_qkv(layout, n, grid, txt, seed):
    """Inputs with block-level structure (a per-block offset) so that block scores differ clearly."""
    t, h, w = grid
    s = t * h * w + txt
    g = torch.Generator().manual_seed(seed)
    base = torch.randn(1, n, s, 128, generator=g)
    centers = torch.randn(1, n, (s + 127) // 128, 128, generator=g).repeat_interleave(128, dim=2)[:, :, :s] * 0.7
    x = base * 0.6 + centers
    q = x.to(torch.bfloat16)
    k = (x * 0.9 + 0.3 * torch.randn(1, n, s, 128, generator=g)).to(torch.bfloat16)
    v = torch.randn(1, n, s, 128, generator=g).to(torch.bfloat16)
    if layout == "BSND":
        q, k, v = (u.transpose(1, 2).contiguous() for u in (q, k, v))
    return q, k, v


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid,txt,sparsity,protect", [
    ("div", 0, 0.0, True), ("div", 0, 0.5, True), ("nodiv_both", 0, 0.75, True), ("nodiv_both", 0, 0.8, False),
    ("nodiv_h", 256, 0.6, True), ("nodiv_w", 100, 0.9, True)])
def test_block_mask_bit_exact(cuda, grid, txt, sparsity, protect, layout):
    from mindiesd.layers.flash_attn import rainfusion as rf
    g3 = GRIDS[grid]
    q, k, v = _structured_qkv(layout, 3, g3, txt, seed=17)
    scale = 128 ** -0.5
    *_, pool = orf.do_tensor_rearrange_pooling(q, k, v, txt, 128, g3, g3, layout)
    want = orf.get_blockwise_mask(pool, txt, sparsity, scale, 128, g3, g3, layout, return_binary=True,
                                  protect_first_frame=protect)
    got = rf.get_blockwise_mask(pool.to(cuda), txt, sparsity, scale, 128, g3, g3, layout, return_binary=True,
                                protect_first_frame=protect)
    assert got.dtype == torch.int8 and got.shape == want.shape
    assert torch.equal(got.cpu(), want), f"{(got.cpu() != want).sum().item()} mask entries differ"
    # every row keeps at least ceil(cols * (1 - sparsity)) blocks (ties and forced blocks add more)
    assert int(got.sum(-1).min()) >= math.ceil(want.shape[-1] * (1 - sparsity))
    # index-list form (rf_v2): same selection, ascending, -1 padded
    sel, num = rf.get_blockwise_mask(pool.to(cuda), txt, sparsity, scale, 128, g3, g3, layout,
                                     protect_first_frame=protect)
    wsel, wnum = orf.get_blockwise_mask(pool, txt, sparsity, scale, 128, g3, g3, layout, protect_first_frame=protect)
    assert sel.dtype == torch.int64 and torch.equal(sel.cpu(), wsel) and torch.equal(num.cpu(), wnum)


def test_block_mask_keep_diagonal_and_fp16(cuda):
    from mindiesd.layers.flash_attn import rainfusion as rf
    g3 = GRIDS["nodiv_both"]
    q, k, v = (u.to(torch.float16) for u in _structured_qkv("BNSD", 2, g3, 0, seed=23))
    *_, pool = orf.do_tensor_rearrange_pooling(q, k, v, 0, 128, g3, g3, "BNSD")
    want = orf.get_blockwise_mask(pool, 0, 0.75, 0.1, 128, g3, g3, "BNSD", return_binary=True, keep_diagonal=True)
    got = rf.get_blockwise_mask(pool.to(cuda), 0, 0.75, 0.1, 128, g3, g3, "BNSD", return_binary=True,
                                keep_diagonal=True)
    assert torch.equal(got.cpu(), want)
    assert bool(torch.diagonal(got, dim1=-2, dim2=-1).all())


def test_get_mask_index_known_answers(cuda):
    """Reference KATs (test_sparse_flash_attn_rf_v2.py:198-216)."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    m = torch.zeros(1, 1, 4, 4, dtype=torch.bool)
    m[0, 0, 0, 0] = m[0, 0, 0, 2] = True
    pos = rf.get_mask_index(m.to(cuda)).cpu()
    assert pos.dtype == torch.int64 and pos[0, 0, 0].tolist() == [0, 2, -1, -1] and pos[0, 0, 1].tolist() == [-1] * 4
    ones = rf.get_mask_index(torch.ones(1, 2, 8, 8, dtype=torch.bool, device=cuda)).cpu()
    assert all(ones[0, n, r].tolist() == list(range(8)) for n in range(2) for r in range(8))


def _random_block_mask(b, n, qb, kb, sparsity, seed):
    g = torch.Generator().manual_seed(seed)
    m = (torch.rand(b, n, qb, kb, generator=g) > sparsity).to(torch.int8)
    m[:, :, 1, :] = 0          # an empty query block must give zeros
    m[:, :, 0, :] = 1
    return m


@pytest.mark.parametrize("s,dtype", [(1024, torch.bfloat16), (1100, torch.bfloat16), (900, torch.float16)])
def test_block_sparse_attention_op_vs_oracle(cuda, s, dtype):
    import mindiesd  # noqa: F401
    q, k, v = (_rand((1, 2, s, 128), seed=i, dtype=dtype) for i in (4, 5, 6))
    nb = (s + 127) // 128
    mask = _random_block_mask(1, 2, nb, nb, 0.5, seed=42)
    scale = 128 ** -0.5
    want = block_sparse_attention(q, k, v, mask, scale)
    out, lse = torch.ops.mindiesd.block_sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), mask.to(cuda),
                                                         scale_value=scale, actual_seq_lengths=[s],
                                                         actual_seq_lengths_kv=[s], softmax_lse_flag=1)
    assert out.dtype == dtype and lse.shape == (1, 2, s, 1) and lse.dtype == torch.float32
    eb, ok, mx = ref_compare(want, out.cpu(), 2 ** -6)
    assert ok, f"mean rel err {eb}, max abs err {mx}"
    assert (out[:, :, 128:256] == 0).all(), "query block with no selected key block must be zero"


def test_block_sparse_dispatch_order_table(cuda):
    """The optional work-order table of the C entry point only changes which workgroup takes which query block:
    any permutation gives the bits of the default order (27 query blocks, not a multiple of the 8 XCDs)."""
    from mindiesd import _native
    from mindiesd.layers.flash_attn import rainfusion as rf
    from mindiesd.layers.flash_attn.hip_flash_attn import _strides_bns
    s, n = 1100, 3
    q, k, v = (_rand((1, n, s, 128), seed=i).to(cuda) for i in (14, 15, 16))
    nb = (s + 127) // 128
    idx, cnt = rf.mask_to_lists(_random_block_mask(1, n, nb, nb, 0.5, seed=7).to(cuda))
    want = rf.block_sparse_attention_lists(q, k, v, idx, cnt, 128 ** -0.5, "BNSD")
    g = torch.Generator().manual_seed(3)
    for order in (torch.randperm(n * nb, generator=g), torch.arange(n * nb - 1, -1, -1)):
        order = order.to(torch.int32).to(cuda)
        out = torch.full_like(q, float("nan"))
        with torch.cuda.device(cuda):
            rc = _native.lib().mindiesd_block_sparse_attention_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), None, _native.DTYPE_CODE[q.dtype], 1, n, n, s, s,
                128, *_strides_bns(q, "BNSD"), *_strides_bns(k, "BNSD"), *_strides_bns(v, "BNSD"),
                *_strides_bns(out, "BNSD"), 128 ** -0.5, idx.data_ptr(), cnt.data_ptr(), idx.shape[3], order.data_ptr(),
                _native.stream_ptr(cuda))
        assert rc == 0
        assert torch.equal(out, want)


def test_full_mask_equals_dense(cuda):
    """sparsity 0 == dense attention (tests/layers/flash_attn/test_sparse_attention.py:73-122)."""
    import mindiesd
    s = 9600
    q, k, v = (_rand((1, s, 3, 128), seed=i) for i in (7, 8, 9))
    dense = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda))
    for st in ("rf_v2", "rf_v3"):
        sp = mindiesd.sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), head_num=3, input_layout="BSND",
                                       sparse_type=st, latent_shape_q=(3, 40, 80), latent_shape_k=(3, 40, 80),
                                       sparsity=0.0)
        eb, ok, mx = ref_compare(dense.cpu(), sp.cpu(), 2 ** -6)
        assert ok, f"{st}: mean rel err {eb}, max abs err {mx}"
    none = mindiesd.sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), head_num=3, input_layout="BSND")
    assert torch.equal(none, dense)


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid", ["div", "nodiv_both"])
def test_rf_v3_end_to_end_vs_oracle(cuda, grid, layout):
    from mindiesd.layers.flash_attn.rainfusion import bsa_sparse_attention_v3
    g3 = GRIDS[grid]
    q, k, v = _structured_qkv(layout, 2, g3, 0, seed=31)
    want, wmask = orf.bsa_sparse_attention_v3(q, k, v, g3, sparsity=0.7, input_layout=layout)
    out, mask = bsa_sparse_attention_v3(q.to(cuda), k.to(cuda), v.to(cuda), g3, sparsity=0.7, input_layout=layout)
    assert torch.equal(mask.cpu(), wmask)
    assert out.shape == q.shape and out.dtype == q.dtype
    eb, ok, mx = ref_compare(want, out.cpu(), 2 ** -6)
    assert ok, f"mean rel err {eb}, max abs err {mx}"
    # cached mask: same result without pooling / mask generation
    out2, mask2 = bsa_sparse_attention_v3(q.to(cuda), k.to(cuda), v.to(cuda), g3, sparsity=0.7, input_layout=layout,
                                          cached_mask=mask)
    assert mask2 is mask and torch.equal(out2, out)


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid,txt", [("div", 0), ("nodiv_both", 0), ("nodiv_h", 256), ("nodiv_w", 128)])
def test_fused_permutation_equals_explicit_passes(cuda, grid, txt, layout):
    """The end-to-end call reads q, k, v and writes the output through the window-order table; the explicit
    chain permute+pool -> mask -> attention -> inverse permute (the reference's sequence of calls,
    rf_v3.py:248-295) must give the same mask and bit-identical output."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    g3 = GRIDS[grid]
    q, k, v = (t.to(cuda) for t in _structured_qkv(layout, 2, g3, txt, seed=77))
    tok = rf.token_order(g3, txt, cuda)
    want_tok = torch.cat([torch.as_tensor(orf.window_order(*g3)) + txt, torch.arange(txt)]).to(torch.int32)
    assert torch.equal(tok.cpu(), want_tok)
    out, mask = rf.bsa_sparse_attention_v3(q, k, v, g3, txt_len=txt, sparsity=0.7, input_layout=layout,
                                           keep_diagonal=True)
    q_, k_, v_, pool = rf.do_tensor_rearrange_pooling(q, k, v, txt, 128, g3, g3, layout)
    mask_x = rf.get_blockwise_mask(pool, txt, 0.7, 128 ** -0.5, 128, g3, g3, layout, return_binary=True,
                                   keep_diagonal=True)
    out_x = rf.rain_fusion_attention_v3(q_, k_, v_, mask_x, input_layout=layout)
    out_x = rf.do_tensor_inv_rearrange(out_x, txt, g3, g3, layout)
    assert torch.equal(mask, mask_x)
    assert torch.equal(out, out_x)


def test_rf_v2_equals_rf_v3(cuda):
    import mindiesd
    g3 = GRIDS["nodiv_w"]
    q, k, v = _structured_qkv("BNSD", 2, g3, 0, seed=37)
    args = dict(head_num=2, input_layout="BNSD", latent_shape_q=g3, latent_shape_k=g3, sparsity=0.6)
    a = mindiesd.sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), sparse_type="rf_v2", **args)
    b = mindiesd.sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), sparse_type="rf_v3", **args)
    assert torch.equal(a, b)


def test_op_argument_errors(cuda):
    import mindiesd  # noqa: F401
    q = torch.randn(1, 2, 256, 128, dtype=torch.bfloat16, device=cuda)
    m = torch.ones(1, 2, 2, 2, dtype=torch.int8, device=cuda)
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.block_sparse_attention(q, q, q, m, q_input_layout="BSH")
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.block_sparse_attention(q, q, q, m, q_input_layout="TND", kv_input_layout="TND")
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.rainfusionattention(q, q, q, m.long()[0], m.long()[0, :, :, 0], [128, 128],
                                               q_input_layout="BSND", kv_input_layout="BSND")
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, input_layout="SBH")
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, sparse_type="topk")
    # 160 image + 77 text tokens: the pooled parts make 2 + 1 blocks, the sequence has 2 - the mask cannot fit the
    # attention (rf_v3.py:219 documents text lengths other than 0 as unsupported), so the call is refused
    from mindiesd.layers.flash_attn.rainfusion import bsa_sparse_attention_v3
    x = torch.randn(1, 2, 237, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(mindiesd.ParametersInvalid):
        bsa_sparse_attention_v3(x, x, x, (1, 8, 20), txt_len=77, input_layout="BNSD")
