"""GPU parity of dense attention at head dims other than 128 (the kernel of csrc/flash_attn_hd.hip) vs the CPU oracle.
The shapes of the first test are the ones the reference's own fused-vs-fallback tests run
(tests/layers/flash_attn/test_attn_forward.py:31-169: [2, 32, 16, 64] BSND, [2, 16, 32, 64] BNSD, [2, 5120, 16, 64]).
bf16 tolerance as for head_dim 128: max-abs <= 2e-2 and cosine >= 0.9999."""
import pytest
import torch

from oracle.attention import attention_math, attention_varlen, causal_keep_mask, cosine, data_compare

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.bfloat16, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * mul).to(dtype)


def _check(out, ref, max_abs=2e-2, min_cos=0.9999):
    assert out.shape == ref.shape and out.dtype == ref.dtype
    assert not torch.isnan(out.float()).any()
    err = (out.float() - ref.float()).abs().max().item()
    assert err <= max_abs, f"max-abs {err}"
    assert cosine(out, ref) >= min_cos, f"cosine {cosine(out, ref)}"


@pytest.mark.parametrize("shape,head_first", [((2, 32, 16, 64), False), ((2, 16, 32, 64), True),
                                              ((2, 5120, 16, 64), False)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_test_shapes(cuda, shape, head_first, dtype):
    import mindiesd
    q, k, v = (_rand(shape, 10 + i, dtype) for i in range(3))
    ref = attention_math(q, k, v, None, None, head_first=head_first)
    for op_type in (None, "prompt_flash_attn", "fused_attn_score", "ascend_laser_attention"):
        kw = {} if op_type is None else {"opt_mode": "manual", "op_type": op_type, "layout": "BNSD"}
        out = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), head_first=head_first, **kw).cpu()
        if dtype == torch.float16:
            _check(out, ref, max_abs=2e-3, min_cos=0.99999)
            assert data_compare(out, ref), "reference's data_compare rule"
        else:
            _check(out, ref)


@pytest.mark.parametrize("d", [8, 40, 64, 72, 96, 120, 136, 160, 192, 256])
@pytest.mark.parametrize("s", [1, 97, 700])
def test_every_padded_width(cuda, d, s):
    """Head dims below, at and above each of the three padded widths (64, 128, 256); the softmax scale is the
    default head_dim ** -0.5; grouped-query heads, key length different from the query length."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    skv = s + 61
    q, k, v = _rand((2, 4, s, d), d), _rand((2, 2, skv, d), d + 1), _rand((2, 2, skv, d), d + 2)
    kk, vv = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    ref = attention_math(q, kk, vv, None, d ** -0.5, head_first=True)
    out, lse = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD", return_lse=True)
    _check(out.cpu(), ref)
    scores = (q.float() @ kk.float().transpose(-1, -2)) * d ** -0.5
    assert (lse.cpu() - torch.logsumexp(scores, dim=-1)).abs().max() < 1e-2


@pytest.mark.parametrize("d", [64, 80, 256])
def test_strided_layouts_run_in_place(cuda, d):
    """BSND storage viewed as BNSD and a BSH-style packed tensor: strides only, no copies."""
    import mindiesd
    q, k, v = (_rand((1, 333, 5, d), 20 + i) for i in range(3))
    ref = attention_math(q, k, v, None, None, head_first=False)
    dev = [t.to(cuda) for t in (q, k, v)]
    out1 = mindiesd.attention_forward(*dev, head_first=False)
    out2 = mindiesd.attention_forward(*(t.transpose(1, 2) for t in dev), head_first=True)
    _check(out1.cpu(), ref)
    assert torch.equal(out1, out2.transpose(1, 2))


@pytest.mark.parametrize("d", [64, 96, 192])
@pytest.mark.parametrize("sq,skv", [(256, 256), (77, 500), (500, 77), (300, 1000)])
def test_causal_and_mask(cuda, d, sq, skv):
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    q, k, v = _rand((1, 2, sq, d), 30), _rand((1, 2, skv, d), 31), _rand((1, 2, skv, d), 32)
    keep = causal_keep_mask(sq, skv)
    rows = keep.any(dim=1)
    ref = attention_math(q[:, :, rows], k, v, keep[rows][None, None].expand(1, 2, -1, -1), d ** -0.5, head_first=True)
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD", causal=True).cpu()
    _check(out[:, :, rows], ref)
    assert not out[:, :, ~rows].any(), "rows without a visible key are zeros"
    g = torch.Generator().manual_seed(33)
    mask = torch.rand((1, 2, sq, skv), generator=g) > 0.5
    mask[..., 3] = True
    ref = attention_math(q, k, v, mask, d ** -0.5, head_first=True)
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD", attn_mask=mask.to(cuda)).cpu()
    _check(out, ref)
    # one mask row shared by all queries (key padding), passed with stride 0 over the queries
    pad = torch.ones(1, 1, 1, skv, dtype=torch.bool)
    pad[..., skv // 2:] = False
    ref = attention_math(q, k, v, pad.expand(1, 2, sq, skv), d ** -0.5, head_first=True)
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD",
                          attn_mask=pad.to(cuda).expand(1, 1, sq, skv)).cpu()
    _check(out, ref)


@pytest.mark.parametrize("d", [64, 72])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen(cuda, d, causal):
    import mindiesd
    lens_q, lens_k = [100, 1, 257, 64], [130, 5, 257, 300]
    cu_q = [0] + torch.tensor(lens_q).cumsum(0).tolist()
    cu_k = [0] + torch.tensor(lens_k).cumsum(0).tolist()
    q, k, v = _rand((cu_q[-1], 4, d), 40), _rand((cu_k[-1], 2, d), 41), _rand((cu_k[-1], 2, d), 42)
    ref = attention_varlen(q, k, v, cu_q, cu_k, None, causal=causal)
    out = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu_q, cu_k, causal=causal).cpu()
    _check(out, ref)
    cu_q_d, cu_k_d = (torch.tensor(c, dtype=torch.int32, device=cuda) for c in (cu_q, cu_k))
    out2 = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu_q_d, cu_k_d, causal=causal).cpu()
    # (host lists size the launch by the longest sequence, device tables by the average: the two may take different
    # kernels, equal up to the summation order)
    assert (out.float() - out2.float()).abs().max() <= 2.0 ** -7
    _check(out2, ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sq,skv", [(2311, 3001), (256, 128), (257, 129), (33, 4100)])
def test_head_dim_64_dense_kernel_against_general_kernel_and_oracle(cuda, sq, skv, dtype):
    """Dense head_dim 64 without a mask runs on its own kernel (csrc/flash_attn_d64.hip); an all-true mask sends the
    same inputs through the general kernel.  Query and key lengths off every tile boundary, grouped-query heads,
    BSND storage; sampled rows against the oracle, everything (and the log-sum-exp) against the general kernel."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    q, k, v = _rand((1, sq, 6, 64), 50, dtype), _rand((1, skv, 2, 64), 51, dtype), _rand((1, skv, 2, 64), 52, dtype)
    dq, dk, dv = q.to(cuda), k.to(cuda), v.to(cuda)
    out, lse = flash_attention(dq, dk, dv, 0.125, "BSND", return_lse=True)
    gen, lse_g = flash_attention(dq, dk, dv, 0.125, "BSND", return_lse=True,
                                 attn_mask=torch.ones(sq, skv, dtype=torch.bool, device=cuda))
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-3
    assert (out.float() - gen.float()).abs().max().item() <= tol
    assert (lse - lse_g).abs().max().item() < 1e-3
    rows = sorted({0, 1, 15, 16, 31, 32, sq // 2, sq - 2, sq - 1} & set(range(sq)))
    kk, vv = k.repeat_interleave(3, dim=2), v.repeat_interleave(3, dim=2)
    ref = attention_math(q[:, rows], kk, vv, None, 0.125, head_first=False)
    _check(out[:, rows].cpu(), ref, max_abs=tol, min_cos=0.9999 if dtype == torch.bfloat16 else 0.99999)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [8, 40, 56, 72, 88, 96, 120])
@pytest.mark.parametrize("sq,skv", [(2311, 3001), (33, 4100), (600, 385)])
def test_head_dims_below_128_on_the_dense_kernels(cuda, d, sq, skv, dtype):
    """Dense attention without a mask at these head dims runs as head_dim 64 (below 64) or 128 (above) on the 16x16x32
    kernels; an all-true mask sends the same inputs through the general kernel.  q, k, v are views of 64- / 128-wide
    buffers whose columns past the head_dim hold NaN: nothing beyond a row's own elements may reach the result.
    Grouped-query heads, BSND storage."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    def in_nan_buffer(t):
        buf = torch.full(t.shape[:-1] + (64 if d < 64 else 128,), float("nan"), dtype=t.dtype, device=cuda)
        buf[..., :d] = t.to(cuda)
        return buf[..., :d]
    q, k, v = _rand((1, sq, 6, d), 70, dtype), _rand((1, skv, 2, d), 71, dtype), _rand((1, skv, 2, d), 72, dtype)
    dq, dk, dv = in_nan_buffer(q), in_nan_buffer(k), in_nan_buffer(v)
    out, lse = flash_attention(dq, dk, dv, d ** -0.5, "BSND", return_lse=True)
    assert not torch.isnan(out.float()).any()
    gen, lse_g = flash_attention(dq, dk, dv, d ** -0.5, "BSND", return_lse=True,
                                 attn_mask=torch.ones(sq, skv, dtype=torch.bool, device=cuda))
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-3
    assert (out.float() - gen.float()).abs().max().item() <= tol
    assert (lse - lse_g).abs().max().item() < 1e-3
    rows = sorted({0, 1, 15, 16, 31, 32, sq // 2, sq - 2, sq - 1} & set(range(sq)))
    kk, vv = k.repeat_interleave(3, dim=2), v.repeat_interleave(3, dim=2)
    ref = attention_math(q[:, rows], kk, vv, None, d ** -0.5, head_first=False)
    _check(out[:, rows].cpu(), ref, max_abs=tol, min_cos=0.9999 if dtype == torch.bfloat16 else 0.99999)
    # contiguous tensors (rows d elements apart: the 256-byte fetch of a row overlaps the next rows) give the same
    out_c = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BSND")
    assert torch.equal(out_c, out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [136, 160, 192, 248, 256])
@pytest.mark.parametrize("sq,skv", [(2311, 3001), (33, 4100), (600, 385)])
def test_head_dims_above_128_on_their_dense_kernel(cuda, d, sq, skv, dtype):
    """Dense attention without a mask at head dims above 128 runs on a kernel of the 128-wide design with 512-byte rows
    (csrc/flash_attn_d256.hip; widths below 256 are computed as 256); an all-true mask sends the same inputs through
    the general kernel.  q, k, v are views of 256-wide buffers whose columns past the head_dim hold NaN: nothing
    beyond a row's own elements may reach the result.  Grouped-query heads, BSND storage."""
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    def in_nan_buffer(t):
        buf = torch.full(t.shape[:-1] + (256,), float("nan"), dtype=t.dtype, device=cuda)
        buf[..., :d] = t.to(cuda)
        return buf[..., :d]
    q, k, v = _rand((1, sq, 4, d), 90, dtype), _rand((1, skv, 2, d), 91, dtype), _rand((1, skv, 2, d), 92, dtype)
    dq, dk, dv = in_nan_buffer(q), in_nan_buffer(k), in_nan_buffer(v)
    out, lse = flash_attention(dq, dk, dv, d ** -0.5, "BSND", return_lse=True)
    assert not torch.isnan(out.float()).any()
    gen, lse_g = flash_attention(dq, dk, dv, d ** -0.5, "BSND", return_lse=True,
                                 attn_mask=torch.ones(sq, skv, dtype=torch.bool, device=cuda))
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-3
    assert (out.float() - gen.float()).abs().max().item() <= tol
    # (both sums are taken over probabilities rounded to 16 bits against different reference maxima: 64- and 32-key tiles)
    assert (lse - lse_g).abs().max().item() < 3e-3
    rows = sorted({0, 1, 15, 16, 31, 32, sq // 2, sq - 2, sq - 1} & set(range(sq)))
    kk, vv = k.repeat_interleave(2, dim=2), v.repeat_interleave(2, dim=2)
    ref = attention_math(q[:, rows], kk, vv, None, d ** -0.5, head_first=False)
    _check(out[:, rows].cpu(), ref, max_abs=tol, min_cos=0.9999 if dtype == torch.bfloat16 else 0.99999)
    out_c = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BSND")
    assert torch.equal(out_c, out)


def test_rejected_head_dims(cuda):
    import mindiesd
    from mindiesd.utils.exception import ParametersInvalid
    for d in (4, 20, 264):
        q = torch.zeros(1, 2, 16, d, dtype=torch.bfloat16, device=cuda)
        with pytest.raises(ParametersInvalid):
            mindiesd.attention_forward(q, q, q, head_first=True)
