"""GPU parity of the general mode of the flash-attention kernel (boolean attention mask, bottom-right aligned
causal mask, packed variable-length sequences) vs the CPU oracle; bf16 tolerance as for the dense kernel:
max-abs <= 2e-2 and cosine >= 0.9999."""
import pytest
import torch

from oracle.attention import attention_math, attention_varlen, causal_keep_mask, cosine

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "256"])
def dense_tile_rows(request, monkeypatch):
    """Causal calls at head_dim 128 choose between the 256-row general kernel and the 128-row one from how the grid
    fills the chip; every test of this file runs under that choice and with the 256-row kernels forced (these small
    grids would not reach them otherwise)."""
    if request.param == "auto":
        monkeypatch.delenv("MINDIESD_DENSE_TILE_ROWS", raising=False)
    else:
        monkeypatch.setenv("MINDIESD_DENSE_TILE_ROWS", request.param)


def _rand(shape, seed, dtype=torch.bfloat16, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * mul).to(dtype)


def _check(out, ref, max_abs=2e-2, min_cos=0.9999):
    assert not torch.isnan(out.float()).any()
    err = (out.float() - ref.float()).abs().max().item()
    assert err <= max_abs, f"max-abs {err}"
    assert cosine(out, ref) >= min_cos, f"cosine {cosine(out, ref)}"


@pytest.mark.parametrize("head_first", [True, False])
@pytest.mark.parametrize("mask_shape", ["2d", "b1", "bn"])
def test_fused_attention_with_boolean_mask(cuda, mask_shape, head_first):
    import mindiesd
    b, n, sq, skv = 2, 3, 300, 421
    q = _rand((b, n, sq, 128), 1)
    k = _rand((b, n, skv, 128), 2)
    v = _rand((b, n, skv, 128), 3)
    g = torch.Generator().manual_seed(4)
    shape = {"2d": (sq, skv), "b1": (b, 1, sq, skv), "bn": (b, n, sq, skv)}[mask_shape]
    mask = torch.rand(shape, generator=g) > 0.4
    mask[..., 5] = True  # every row keeps at least one key
    full = mask if mask.dim() == 4 else mask[None, None]
    ref = attention_math(q, k, v, full.expand(b, n, sq, skv), head_first=True)
    args = (q, k, v) if head_first else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = mindiesd.attention_forward(*(t.to(cuda) for t in args), attn_mask=mask.to(cuda), head_first=head_first).cpu()
    _check(out if head_first else out.transpose(1, 2), ref)


def test_mask_hides_the_first_tiles_and_scores_lie_far_below_zero(cuda):
    """Block-diagonal mask (rows of the second half see keys of the second half only, so their first two key tiles are
    hidden) on scores hundreds of units below zero: a row must take its reference maximum from the first tile that
    shows it a key.  fp64 yardstick on the queries as the kernel rounds them (q * scale * log2(e) in bf16)."""
    import math
    import mindiesd
    from oracle.attention import attention_fp64
    s = 600
    g = torch.Generator().manual_seed(9)
    q = (8.0 + 0.5 * torch.randn((1, 2, s, 128), generator=g)).to(torch.bfloat16)
    k = (-8.0 + 0.5 * torch.randn((1, 2, s, 128), generator=g)).to(torch.bfloat16)
    v = torch.randn((1, 2, s, 128), generator=g).to(torch.bfloat16)
    mask = torch.zeros(s, s, dtype=torch.bool)
    mask[:300, :300] = True
    mask[300:, 300:] = True
    out = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask.to(cuda), head_first=True).cpu()
    qs = (q.float() * (128 ** -0.5 * math.log2(math.e))).to(torch.bfloat16)
    for n in range(2):
        _check(out[0, n], attention_fp64(qs[0, n], k[0, n], v[0, n], math.log(2.0), keep=mask.numpy()))


def test_mask_dtypes_and_fully_masked_rows(cuda):
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    q, k, v = _rand((1, 2, 130, 128), 5), _rand((1, 2, 200, 128), 6), _rand((1, 2, 200, 128), 7)
    mask = torch.zeros(130, 200, dtype=torch.int32)
    mask[:, 17] = 3          # non-zero = attend
    mask[7] = 0              # a row without any visible key
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), 128 ** -0.5, "BNSD", attn_mask=mask.to(cuda)).cpu()
    assert not out[:, :, 7].any()
    rows = [r for r in range(130) if r != 7]
    assert torch.equal(out[:, :, rows], v[:, :, 17:18].expand(1, 2, 129, 128))  # one visible key: the output is its value row


# (from 256 query rows on, calls without a mask run on the 8-wave kernel's general instantiation)
@pytest.mark.parametrize("sq,skv", [(256, 256), (300, 300), (77, 500), (500, 77), (1000, 1300), (1100, 1100),
                                    (1300, 1800), (1800, 1300), (1025, 2047), (1536, 385)])
def test_causal_bottom_right(cuda, sq, skv):
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    q, k, v = _rand((1, 4, sq, 128), 8), _rand((1, 2, skv, 128), 9), _rand((1, 2, skv, 128), 10)
    out, lse = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), 128 ** -0.5, "BNSD", return_lse=True, causal=True)
    keep = causal_keep_mask(sq, skv)
    kk, vv = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    ref = attention_math(q, kk, vv, keep, head_first=True)
    seen = keep.any(-1)
    ref = torch.where(seen[None, None, :, None], ref, torch.zeros((), dtype=ref.dtype))
    _check(out.cpu(), ref)
    assert not out.cpu()[:, :, ~seen].any()
    s = (q.float() @ kk.float().transpose(-1, -2)) * 128 ** -0.5
    want_lse = torch.logsumexp(s.masked_fill(~keep, float("-inf")), dim=-1)
    assert torch.allclose(lse.cpu()[:, :, seen], want_lse[:, :, seen], atol=5e-3, rtol=0)
    assert torch.isinf(lse.cpu()[:, :, ~seen]).all()


@pytest.mark.parametrize("d", [128, 64, 96, 40, 160, 256])
@pytest.mark.parametrize("sq,skv", [(1100, 1100), (1300, 1800), (1800, 1300), (2049, 2049)])
def test_causal_long_sequences_head_dims(cuda, sq, skv, d):
    """The causal instantiations of the two 16x16x32 kernels (head_dim 128 and 64; 96 and 40 run padded on them), three
    heads (heavy and light tiles are dealt to the XCDs in pairs: an odd and an even tile count)."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    q, k, v = _rand((2, 3, sq, d), 8), _rand((2, 3, skv, d), 9), _rand((2, 3, skv, d), 10)
    out, lse = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD", return_lse=True, causal=True)
    keep = causal_keep_mask(sq, skv)
    ref = attention_math(q, k, v, keep, d ** -0.5, head_first=True)
    seen = keep.any(-1)
    ref = torch.where(seen[None, None, :, None], ref, torch.zeros((), dtype=ref.dtype))
    _check(out.cpu(), ref)
    assert not out.cpu()[:, :, ~seen].any()
    s = (q.float() @ k.float().transpose(-1, -2)) * d ** -0.5
    want_lse = torch.logsumexp(s.masked_fill(~keep, float("-inf")), dim=-1)
    # (the kernel rounds q * scale * log2(e) to 16 bits: 2^-9 of a score that a row with few keys consists of)
    assert torch.allclose(lse.cpu()[:, :, seen], want_lse[:, :, seen], atol=1e-2, rtol=0)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_forward_varlen(cuda, causal):
    import mindiesd
    lens_q, lens_k = [300, 1, 0, 513, 40], [300, 77, 5, 256, 900]
    cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
    q, k, v = _rand((sum(lens_q), 4, 128), 11), _rand((sum(lens_k), 2, 128), 12), _rand((sum(lens_k), 2, 128), 13)
    out = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu_q.to(cuda), cu_k.to(cuda),
                                            causal=causal).cpu()
    ref = attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), causal=causal)
    assert out.shape == q.shape and out.dtype == q.dtype
    _check(out, ref)
    # lists of python ints work as well, and a custom scale
    out2 = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu_q.tolist(), cu_k.tolist(),
                                             softmax_scale=0.05, causal=causal).cpu()
    _check(out2, attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), scale=0.05, causal=causal))


def test_varlen_device_table_uncovered_rows_and_named_bounds(cuda):
    """Device cu_seqlens cannot be validated without a host read-back: rows that no sequence covers come back as
    zeros (not as whatever the allocation held), and the optional longest-sequence bounds give the same result."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention_varlen
    lens = [200, 150]                                 # 350 of 400 query tokens are covered
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    q, k, v = _rand((400, 2, 128), 21), _rand((350, 2, 128), 22), _rand((350, 2, 128), 23)
    torch.full((400, 2, 128), float("nan"), dtype=torch.bfloat16, device=cuda)   # dirty the allocator's pool
    torch.cuda.empty_cache()
    out = flash_attention_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu.to(cuda), cu.to(cuda), 128 ** -0.5).cpu()
    ref = attention_varlen(q[:350], k, v, cu.tolist(), cu.tolist())
    _check(out[:350], ref)
    assert (out[350:] == 0).all()
    out2 = flash_attention_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu.to(cuda), cu.to(cuda), 128 ** -0.5,
                                  max_seqlen_q=200, max_seqlen_k=200).cpu()
    assert torch.equal(out2, out)


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen_many_sequences_device_table(cuda, d, causal):
    """150 sequences (more than one wave's worth of table entries) of lengths 0 .. 300, key lengths different from the
    query lengths, cu_seqlens on the device: the packed entry point numbers the query tiles through the sequences.
    Same result as with the host lists (which size the grid by the longest sequence) and parity with the oracle."""
    import random
    import mindiesd
    r = random.Random(d + causal)
    lens_q = [r.choice([0, 1, 5, 127, 128, 129, 200, 300]) for _ in range(150)]
    lens_k = [max(1, l + r.choice([-3, 0, 0, 40])) for l in lens_q]
    cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
    q, k, v = _rand((sum(lens_q), 2, d), 61), _rand((sum(lens_k), 1, d), 62), _rand((sum(lens_k), 1, d), 63)
    dev = [t.to(cuda) for t in (q, k, v)]
    out_dev = mindiesd.attention_forward_varlen(*dev, cu_q.to(cuda), cu_k.to(cuda), causal=causal).cpu()
    out_host = mindiesd.attention_forward_varlen(*dev, cu_q.tolist(), cu_k.tolist(), causal=causal).cpu()
    # (host lists size the launch by the longest sequence, device tables by the average: the two may take different
    # kernels, equal up to the summation order)
    assert (out_dev.float() - out_host.float()).abs().max() <= 2.0 ** -6
    _check(out_dev, attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), causal=causal))


@pytest.mark.parametrize("d", [128, 64, 96, 40, 160, 256])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_varlen_long_sequences(cuda, causal, dtype, d):
    """Long sequences on the 8-wave kernel (256-row tiles): lengths around the tile edges,
    key counts above and below the query counts (causal rows without any visible key give zeros), a sequence without
    keys and one without queries, grouped heads.  Host lists size the grid by the longest sequence; device tables
    of long sequences number the tiles through the table."""
    # (values of 0.5 * N(0, 1): a causal row's first keys give outputs that are single value rows, and above 2 one bf16
    # step is 2^-6, most of the tolerance)
    import mindiesd
    lens_q, lens_k = [1500, 1, 0, 1100, 300, 40, 1281], [1500, 700, 5, 1300, 2000, 0, 1000]
    cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
    q, k, v = (_rand((sum(lens_q), 4, d), 31, dtype), _rand((sum(lens_k), 2, d), 32, dtype),
               _rand((sum(lens_k), 2, d), 33, dtype, mul=0.5))
    ref = attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), causal=causal)
    dev = [t.to(cuda) for t in (q, k, v)]
    out = mindiesd.attention_forward_varlen(*dev, cu_q.tolist(), cu_k.tolist(), causal=causal).cpu()
    _check(out, ref)
    o5 = int(cu_q[5])
    assert not out[o5:o5 + 40].any()          # the sequence without keys
    # device tables: 4 long sequences (average >= 1024 tokens), tiles numbered through the table
    lq2, lk2 = [1500, 1100, 1281, 2049], [1500, 1300, 1000, 2049]
    cq2 = torch.tensor([0] + lq2).cumsum(0).to(torch.int32)
    ck2 = torch.tensor([0] + lk2).cumsum(0).to(torch.int32)
    q2, k2, v2 = (_rand((sum(lq2), 4, d), 34, dtype), _rand((sum(lk2), 2, d), 35, dtype),
                  _rand((sum(lk2), 2, d), 36, dtype, mul=0.5))
    dev2 = [t.to(cuda) for t in (q2, k2, v2)]
    out_dev = mindiesd.attention_forward_varlen(*dev2, cq2.to(cuda), ck2.to(cuda), causal=causal).cpu()
    out_host = mindiesd.attention_forward_varlen(*dev2, cq2.tolist(), ck2.tolist(), causal=causal).cpu()
    # (host lists size the launch by the longest sequence, device tables by the average: the two may take different
    # kernels, equal up to the summation order)
    assert (out_dev.float() - out_host.float()).abs().max() <= 2.0 ** -6
    _check(out_dev, attention_varlen(q2, k2, v2, cq2.tolist(), ck2.tolist(), causal=causal))


@pytest.mark.parametrize("d", [128, 64, 96, 40, 160, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen_many_long_sequences_device_table(cuda, d, causal):
    """70 sequences (more than one wave's worth of table entries) of 1024 tokens and more on average, two of them
    empty and one much longer than the rest, cu_seqlens on the device: the packed numbering of the 8-wave kernels."""
    import random
    import mindiesd
    r = random.Random(100 + d + causal)
    lens_q = [r.choice([1024, 1100, 1281, 1536]) for _ in range(70)]
    lens_q[3] = 0
    lens_q[66] = 0
    lens_q[40] = 5000
    lens_k = [max(1, l + r.choice([-300, 0, 0, 257])) for l in lens_q]
    cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
    # (values of 0.5 * N(0, 1): a causal row's first keys give outputs that are single value rows, and above 2 one bf16
    # step is 2^-6, most of the tolerance)
    q, k, v = _rand((sum(lens_q), 2, d), 81), _rand((sum(lens_k), 1, d), 82), _rand((sum(lens_k), 1, d), 83, mul=0.5)
    dev = [t.to(cuda) for t in (q, k, v)]
    out_dev = mindiesd.attention_forward_varlen(*dev, cu_q.to(cuda), cu_k.to(cuda), causal=causal).cpu()
    out_host = mindiesd.attention_forward_varlen(*dev, cu_q.tolist(), cu_k.tolist(), causal=causal).cpu()
    # (host lists size the launch by the longest sequence, device tables by the average: the two may take different
    # kernels, equal up to the summation order)
    assert (out_dev.float() - out_host.float()).abs().max() <= 2.0 ** -6
    _check(out_dev, attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), causal=causal))


def test_varlen_single_sequence_equals_dense(cuda):
    import mindiesd
    q, k, v = _rand((700, 2, 128), 14, mul=0.5), _rand((700, 2, 128), 15, mul=0.5), _rand((700, 2, 128), 16, mul=0.5)
    a = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), [0, 700], [0, 700])
    b = mindiesd.attention_forward(q[None].to(cuda), k[None].to(cuda), v[None].to(cuda))
    # different tile shapes behind the two entry points: equal up to the summation order
    assert (a.float() - b[0].float()).abs().max() <= 2.0 ** -8 and cosine(a, b[0]) >= 0.99999


def test_varlen_and_mask_errors(cuda):
    import mindiesd
    from mindiesd import ParametersInvalid
    q = torch.randn(10, 2, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(ParametersInvalid, match="Unsupported parameters in varlen attention"):
        mindiesd.attention_forward_varlen(q, q, q, [0, 10], [0, 10], window_size=3)
    with pytest.raises(ParametersInvalid, match="dropout_p"):
        mindiesd.attention_forward_varlen(q, q, q, [0, 10], [0, 10], dropout_p=0.1)
    with pytest.raises(ParametersInvalid, match="3D"):
        mindiesd.attention_forward_varlen(q[None], q[None], q[None], [0, 10], [0, 10])
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward_varlen(q, q, q, [0, 9], [0, 10])
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward_varlen(q, q, q, [0, 4, 10], [0, 10])
    x = torch.randn(1, 64, 2, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(ParametersInvalid, match="attn_mask"):
        mindiesd.attention_forward(x, x, x, attn_mask=torch.ones(3, 64, 64, dtype=torch.bool, device=cuda))
    with pytest.raises(ParametersInvalid, match="attn_mask"):
        mindiesd.attention_forward(x, x, x, attn_mask=torch.ones(63, 64, dtype=torch.bool, device=cuda))


def test_key_padding_mask_expanded_over_queries(cuda):
    """[B, 1, 1, Skv] key-padding mask expanded to [B, 1, Sq, Skv]: a view whose query stride is 0 runs without
    being materialised."""
    import mindiesd
    b, n, sq, skv = 2, 2, 260, 333
    q, k, v = _rand((b, n, sq, 128), 21), _rand((b, n, skv, 128), 22), _rand((b, n, skv, 128), 23)
    keep = torch.ones(b, 1, 1, skv, dtype=torch.bool)
    keep[0, ..., 300:] = False
    keep[1, ..., 17:40] = False
    ref = attention_math(q, k, v, keep.expand(b, n, sq, skv), head_first=True)
    view = keep.to(cuda).expand(b, 1, sq, skv)
    assert view.stride(2) == 0
    out = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=view, head_first=True).cpu()
    _check(out, ref)


@pytest.mark.parametrize("d", [128, 64, 96, 40, 160, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("per_head", [False, True])
def test_key_padding_mask_long_sequences(cuda, per_head, dtype, d):
    """From 256 query rows on, a mask row shared by all queries runs on the 8-wave kernel (mask bytes reduced to
    words of visible keys per tile).  Trailing padding, holes, a random half, a row that hides its first two key tiles,
    a batch entry without any visible key (zeros); key count off the tile size, mask rows at odd addresses."""
    import mindiesd
    b, n, sq, skv = 5, 2, 1100, 1355
    q, k, v = _rand((b, n, sq, d), 41, dtype), _rand((b, n, skv, d), 42, dtype), _rand((b, n, skv, d), 43, dtype)
    g = torch.Generator().manual_seed(44)
    keep = torch.ones(b, n if per_head else 1, 1, skv, dtype=torch.bool)
    keep[0, ..., 1000:] = False                       # trailing padding
    keep[1, ..., 17:40] = False                       # holes, one of them a whole tile
    keep[1, ..., 256:384] = False
    keep[2] = torch.rand(keep[2].shape, generator=g) > 0.5
    keep[3, ..., :300] = False                        # the first two tiles hidden
    keep[4] = False                                   # nothing visible
    if per_head:
        keep[0, 1, ..., 500:] = False
    full = keep.expand(b, n, sq, skv)
    ref = attention_math(q, k, v, full, d ** -0.5, head_first=True)
    ref[4] = 0
    view = keep.to(cuda).expand(b, keep.shape[1], sq, skv)
    assert view.stride(2) == 0
    out, lse = mindiesd.layers.flash_attn.hip_flash_attn.flash_attention(
        q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD", attn_mask=view, return_lse=True)
    out = out.cpu()
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-3
    _check(out[:4], ref[:4], max_abs=tol)
    assert not out[4].any()
    s = (q.float() @ k.float().transpose(-1, -2)) * d ** -0.5
    want_lse = torch.logsumexp(s.masked_fill(~full, float("-inf")), dim=-1)
    assert torch.allclose(lse.cpu()[:4], want_lse[:4], atol=5e-3, rtol=0)
    assert torch.isinf(lse.cpu()[4]).all()
    # the same mask without the expansion ([B, N|1, 1, Skv])
    out_b = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=keep.to(cuda), head_first=True).cpu()
    assert torch.equal(out_b, out)
    # the materialised mask takes the general kernel: same result up to the summation order
    out_full = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=full.contiguous().to(cuda),
                                          head_first=True).cpu()
    assert (out.float() - out_full.float()).abs().max() <= tol


def test_key_padding_mask_first_visible_key_far_below_zero(cuda):
    """Scores hundreds of units below zero and a mask that hides the first tiles: the reference maximum must come
    from the first tile that shows a key (fp64 yardstick on the queries as the kernel rounds them)."""
    import math
    import mindiesd
    from oracle.attention import attention_fp64
    sq, skv = 1024, 1500
    g = torch.Generator().manual_seed(45)
    q = (8.0 + 0.5 * torch.randn((1, 2, sq, 128), generator=g)).to(torch.bfloat16)
    k = (-8.0 + 0.5 * torch.randn((1, 2, skv, 128), generator=g)).to(torch.bfloat16)
    v = torch.randn((1, 2, skv, 128), generator=g).to(torch.bfloat16)
    keep = torch.zeros(1, 1, 1, skv, dtype=torch.bool)
    keep[..., 700:1400] = True
    out = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=keep.to(cuda).expand(1, 1, sq, skv),
                                     head_first=True).cpu()
    qs = (q.float() * (128 ** -0.5 * math.log2(math.e))).to(torch.bfloat16)
    m2 = keep[0, 0].expand(sq, skv).numpy()
    for n in range(2):
        _check(out[0, n], attention_fp64(qs[0, n], k[0, n], v[0, n], math.log(2.0), keep=m2))
