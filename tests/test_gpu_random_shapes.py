"""GPU parity on shapes drawn at random (fixed seeds): sequence lengths around every tile and block boundary, unequal
query / key lengths, grouped-query heads, both layouts and dtypes, head dims of every kernel, random boolean masks,
causal masks and random block masks, the MXFP8 GEMM with and without SwiGLU and bias, each against the CPU oracle
with the tolerance of the path's own test file; the two quantisers bit for bit on values spread over many octaves, tiny values, values on a coarse grid (rounding
ties) and outliers."""
import random

import pytest
import torch

from oracle import attention as oa
from oracle.attention import attention_math, causal_keep_mask

pytestmark = pytest.mark.gpu

SQ = [1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 127, 129, 255, 256, 257, 383, 385, 511, 513, 640, 777, 1000]
SKV = [1, 3, 32, 63, 64, 65, 96, 127, 128, 129, 191, 193, 255, 257, 300, 449, 512, 515, 901]


def _rnd(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


def _heads(r):
    n = r.choice([1, 2, 3, 4])
    return n, r.choice([x for x in (1, 2, 3, 4) if n % x == 0])


@pytest.mark.parametrize("seed", range(48))
def test_dense_random_shape(cuda, seed, monkeypatch):
    import mindiesd
    r = random.Random(seed)
    # (head_dim 128: the library picks 256- or 128-row workgroups from how the grid fills the chip; odd seeds force
    # the 256-row kernel, which these small grids would not reach otherwise)
    if seed % 2:
        monkeypatch.setenv("MINDIESD_DENSE_TILE_ROWS", "256")
    d = r.choice([128, 128, 64, 32, 96, 256])
    sq = r.choice(SQ)
    skv = sq if r.random() < 0.5 else r.choice(SKV)
    (n, nkv), b = _heads(r), r.choice([1, 2])
    dtype, hf = r.choice([torch.bfloat16, torch.float16]), r.random() < 0.5
    q, k, v = _rnd((b, n, sq, d), seed, dtype), _rnd((b, nkv, skv, d), seed + 1000, dtype), _rnd((b, nkv, skv, d), seed + 2000, dtype)
    ref = attention_math(q, k.repeat_interleave(n // nkv, 1), v.repeat_interleave(n // nkv, 1), None, d ** -0.5, head_first=True)
    args = (q, k, v) if hf else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = mindiesd.attention_forward(*(t.to(cuda) for t in args), head_first=hf).cpu()
    out = out if hf else out.transpose(1, 2)
    assert not torch.isnan(out.float()).any()
    assert (out.float() - ref.float()).abs().max().item() <= 2e-2, (b, n, nkv, sq, skv, d, dtype, hf)


@pytest.mark.parametrize("seed,case", [(2031, (2, 3, 3, 31, 31, 256)), (2283, (1, 3, 1, 257, 63, 128)),
                                       (2495, (1, 4, 2, 640, 63, 128)), (2871, (2, 1, 1, 777, 3, 256))])
def test_few_keys_against_exact_softmax(cuda, seed, case):
    """Four shapes with few keys (3 .. 63) found by running the test above on 1200 further seeds, where kernel and
    oracle differ by 0.023 .. 0.031 in outputs of magnitude 2: the oracle follows the reference's bf16 roundings of
    q * scale, the scores and the probabilities (attention_func.py:38-50), and with so few keys nothing averages them
    out - it lies 0.017 .. 0.027 from the softmax evaluated in float64 on the same bf16 inputs, the kernel (float32
    scores and sums) 0.005 .. 0.014.  The kernel is held to the 2e-2 bound against the float64 result here, and to
    its distance from the oracle being no more than the oracle's own from that result plus the bound's half."""
    import mindiesd
    b, n, nkv, sq, skv, d = case
    q, k, v = (_rnd((b, n, sq, d), seed, torch.bfloat16), _rnd((b, nkv, skv, d), seed + 1000, torch.bfloat16),
               _rnd((b, nkv, skv, d), seed + 2000, torch.bfloat16))
    kk, vv = k.repeat_interleave(n // nkv, 1), v.repeat_interleave(n // nkv, 1)
    exact = (torch.softmax(q.double() @ kk.double().transpose(-1, -2) * d ** -0.5, -1) @ vv.double()).float()
    ref = attention_math(q, kk, vv, None, d ** -0.5, head_first=True).float()
    out = mindiesd.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), head_first=True).cpu().float()
    assert (out - exact).abs().max().item() <= 2e-2
    assert (out - ref).abs().max().item() <= (ref - exact).abs().max().item() + 1e-2


@pytest.mark.parametrize("seed", range(32))
def test_masked_or_causal_random_shape(cuda, seed):
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    r = random.Random(100 + seed)
    d = r.choice([128, 128, 64])
    sq, skv = r.choice([1, 17, 64, 100, 129, 256, 300, 513]), r.choice([1, 5, 64, 65, 128, 200, 257, 400, 640])
    (n, nkv), b = _heads(r), r.choice([1, 2])
    causal = r.random() < 0.4
    q, k, v = _rnd((b, n, sq, d), seed, torch.bfloat16), _rnd((b, nkv, skv, d), seed + 1, torch.bfloat16), _rnd((b, nkv, skv, d), seed + 2, torch.bfloat16)
    if causal:
        mask, keep = None, causal_keep_mask(sq, skv)[None, None].expand(b, n, sq, skv)
    else:
        g = torch.Generator().manual_seed(seed)
        mask = torch.rand((b, r.choice([1, n]), sq, skv), generator=g) > r.choice([0.2, 0.5, 0.9])
        keep = mask.expand(b, n, sq, skv)
    ref = attention_math(q, k.repeat_interleave(n // nkv, 1), v.repeat_interleave(n // nkv, 1), keep, d ** -0.5, head_first=True)
    ref = torch.where(keep.any(-1)[..., None], ref, torch.zeros((), dtype=ref.dtype))  # rows without a visible key: zeros
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD",
                          attn_mask=None if mask is None else mask.to(cuda), causal=causal).cpu()
    assert not torch.isnan(out.float()).any()
    # A row that sees only a handful of keys is a weighted mean of a few v rows: the rounding of the scores (the
    # reference keeps q * scale and q k^T in bf16, attention_func.py:40-41, the kernel q * scale * log2(e)) moves
    # single weights by a few per cent and nothing averages that out, hence 5e-2 where the dense bound is 2e-2.
    err = (out.float() - ref.float()).abs()
    assert bool((err <= 5e-2 * ref.float().abs().clamp(min=1.0)).all()), (err.max().item(), b, n, nkv, sq, skv, d, causal)
    dense_rows = keep.sum(-1) >= 32
    assert err[dense_rows].max().item() <= 2e-2 if dense_rows.any() else True


@pytest.mark.parametrize("seed", range(40))
def test_long_random_shape(cuda, seed, monkeypatch):
    """Long sequences, where dense, causal, key-mask and packed calls run on the 16x16x32 kernels at every
    head_dim (padded where it is not 64, 128 or 256): random lengths off the tile sizes, head dims of every kernel,
    grouped-query heads, both dtypes."""
    import mindiesd
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    from oracle.attention import attention_varlen
    r = random.Random(300 + seed)
    if seed % 2:
        monkeypatch.setenv("MINDIESD_DENSE_TILE_ROWS", "256")   # (see test_dense_random_shape)
    d = r.choice([40, 64, 72, 96, 128, 128, 160, 256])
    mode = r.choice(["dense", "causal", "keymask", "varlen", "varlen_causal"])
    sq, skv = r.randrange(1024, 2400), r.randrange(385, 2600)
    (n, nkv), b = _heads(r), r.choice([1, 2])
    dtype = r.choice([torch.bfloat16, torch.float16])
    info = (mode, b, n, nkv, sq, skv, d, dtype)
    if mode.startswith("varlen"):
        nseq = r.choice([2, 3, 5])
        lens_q = [r.choice([0, 1, 200, 1024, 1300, r.randrange(1, 2000)]) for _ in range(nseq)]
        lens_q[r.randrange(nseq)] = r.randrange(1024, 2200)            # at least one long sequence
        lens_k = [max(1, l + r.choice([-100, 0, 0, 300])) for l in lens_q]
        cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
        cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
        q, k, v = (_rnd((sum(lens_q), n, d), seed, dtype), _rnd((sum(lens_k), nkv, d), seed + 1, dtype),
                   _rnd((sum(lens_k), nkv, d), seed + 2, dtype) * 0.5)
        causal = mode == "varlen_causal"
        table = (cu_q.to(cuda), cu_k.to(cuda)) if r.random() < 0.5 else (cu_q.tolist(), cu_k.tolist())
        out = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), *table, causal=causal).cpu()
        ref = attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), causal=causal)
        assert not torch.isnan(out.float()).any()
        err = (out.float() - ref.float()).abs()
        assert bool((err <= 5e-2 * ref.float().abs().clamp(min=1.0)).all()), (err.max().item(), info, lens_q, lens_k)
        return
    q, k, v = _rnd((b, n, sq, d), seed, dtype), _rnd((b, nkv, skv, d), seed + 1, dtype), _rnd((b, nkv, skv, d), seed + 2, dtype)
    mask, keep = None, None
    if mode == "causal":
        keep = causal_keep_mask(sq, skv)[None, None].expand(b, n, sq, skv)
    elif mode == "keymask":
        g = torch.Generator().manual_seed(seed)
        mask = torch.rand((b, r.choice([1, n]), 1, skv), generator=g) > r.choice([0.1, 0.5, 0.97])
        if r.random() < 0.5:
            mask[..., :r.randrange(1, skv)] = False                    # the first tiles hidden
        keep = mask.expand(b, n, sq, skv)
    ref = attention_math(q, k.repeat_interleave(n // nkv, 1), v.repeat_interleave(n // nkv, 1), keep, d ** -0.5, head_first=True)
    if keep is not None:
        ref = torch.where(keep.any(-1)[..., None], ref, torch.zeros((), dtype=ref.dtype))
    out = flash_attention(q.to(cuda), k.to(cuda), v.to(cuda), d ** -0.5, "BNSD",
                          attn_mask=None if mask is None else mask.to(cuda), causal=mode == "causal").cpu()
    assert not torch.isnan(out.float()).any()
    err = (out.float() - ref.float()).abs()
    assert bool((err <= 5e-2 * ref.float().abs().clamp(min=1.0)).all()), (err.max().item(), info)
    if keep is None:
        assert err.max().item() <= 2e-2, (err.max().item(), info)
    else:
        dense_rows = keep.sum(-1) >= 32
        assert err[dense_rows].max().item() <= 2e-2 if dense_rows.any() else True, info


@pytest.mark.parametrize("seed", range(24))
def test_block_sparse_random_mask(cuda, seed):
    from mindiesd.layers.flash_attn import rainfusion as rf
    r = random.Random(200 + seed)
    s = r.choice([130, 255, 256, 257, 500, 640, 769, 1024, 1100, 1537])
    n = r.choice([1, 2, 4])
    nkv, b = r.choice([x for x in (1, 2, 4) if n % x == 0]), r.choice([1, 2])
    dtype = r.choice([torch.bfloat16, torch.float16])
    q, k, v = _rnd((b, n, s, 128), seed, dtype), _rnd((b, nkv, s, 128), seed + 1, dtype), _rnd((b, nkv, s, 128), seed + 2, dtype)
    nb = (s + 127) // 128
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(b, n, nb, nb, generator=g) < r.choice([0.1, 0.3, 0.6, 0.9])
    want = oa.block_sparse_attention(q, k, v, m.numpy())
    out = rf.block_sparse_attention_mask(q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda), 128 ** -0.5, "BNSD").cpu()
    assert not torch.isnan(out.float()).any()
    eb, ok, mx = oa.ref_compare(want, out, 2.0 ** -6)
    assert ok, (eb, mx, b, n, nkv, s, dtype)


def _values(shape, seed, dtype, kind):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    if kind == "wide":      # magnitudes over ten octaves of ten, row by row
        x = x * torch.logspace(-6, 4, shape[-2], base=10.0)[:, None]
    elif kind == "tiny":
        x = x * 1e-6
    elif kind == "ties":    # a coarse grid: many values halfway between two codes
        x = torch.round(x * 4) / 4
    elif kind == "outlier":
        x = torch.where(torch.rand(shape, generator=g) < 0.01, x * 50, x)
    x = x.to(dtype)
    return x.clamp(-60000, 60000) if dtype == torch.float16 else x


KINDS = ["normal", "wide", "tiny", "ties", "outlier"]


@pytest.mark.parametrize("seed", range(20))
def test_mx_quant_random(cuda, seed):
    from mindiesd.layers.quant import mx_quantize
    from oracle import quant as oq
    r = random.Random(300 + seed)
    dtype, kind = r.choice([torch.bfloat16, torch.float16]), r.choice(KINDS)
    m, k = r.choice([1, 5, 31, 32, 33, 127, 128, 129, 300, 1000]), r.choice([32, 64, 128, 256, 320, 512, 1024])
    x = _values((m, k), seed, dtype, kind)
    q, e = mx_quantize(x.to(cuda))
    codes, e8 = oq.mx_quant(x)
    got = q.view(torch.uint8).cpu()
    assert torch.equal(e.view(torch.uint8).cpu(), e8), (m, k, dtype, kind)
    assert torch.equal(got & 0x7f, codes & 0x7f), (m, k, dtype, kind)
    assert torch.equal((got >> 7)[codes & 0x7f != 0], (codes >> 7)[codes & 0x7f != 0])  # the sign of a zero is free


@pytest.mark.parametrize("seed", range(20))
def test_block_quant_random(cuda, seed):
    from mindiesd.layers.quant.block_quant import _block_quant
    from oracle import quant as oq
    r = random.Random(400 + seed)
    dtype, kind = r.choice([torch.bfloat16, torch.float16]), r.choice(KINDS)
    s, n = r.choice([1, 100, 127, 128, 129, 256, 300, 1000]), r.choice([1, 2, 3])
    layout, pow2, pre = r.choice(["BNSD", "BSND"]), r.random() < 0.5, r.choice([1.0, 1.0, 0.127, 3.5])
    x = _values((1, n, s, 128), seed, dtype, kind)
    xd = x.to(cuda) if layout == "BNSD" else x.transpose(1, 2).contiguous().to(cuda)
    c, sc = _block_quant(xd, 128, layout, pre, pow2)
    wc, ws = oq.dynamic_block_quant(x, 128, 128, pre, pow2)
    got = c.cpu().view(torch.uint8)
    assert torch.equal(sc.cpu(), ws[..., 0]), (n, s, dtype, kind, layout, pow2, pre)
    zero = ((got & 0x7f) == 0) & ((wc & 0x7f) == 0)
    assert bool(((got == wc) | zero).all()), (n, s, dtype, kind, layout, pow2, pre)


@pytest.mark.parametrize("seed", range(24))
def test_fp8_attention_random_shape(cuda, seed):
    """FP8 attention on random lengths (around every tile boundary, query and key lengths unequal), both layouts and
    dtypes, every combination of scale recipe, probability rule and K block, inputs with and without outliers and with
    rising row maxima: against the oracle that re-quantises the probabilities the way the kernel does."""
    from mindiesd.layers.quant import fp8_attention_forward
    from oracle import quant as oq
    r = random.Random(700 + seed)
    dtype, layout = r.choice([torch.bfloat16, torch.float16]), r.choice(["BNSD", "BSND"])
    sq, skv, n = r.choice(SQ), r.choice([s for s in SKV if s >= 3]), r.choice([1, 2, 3])
    recipe, p_rule, k_block = r.choice(["amax", "pow2"]), r.choice(["linear", "exp2"]), r.choice([128, 256])
    g = torch.Generator().manual_seed(seed)
    def make(s):
        x = torch.randn((1, n, s, 128), generator=g)
        if seed % 3:
            x = torch.where(torch.rand((1, n, s, 128), generator=g) < 0.01, x * 8, x)
        return x.to(dtype)
    q, k, v = make(sq), make(skv), make(skv)
    if seed % 2:
        k[:, :, skv // 2:] *= 1.7                      # the reference maximum has to move late in the row
    want = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", requant_p=True, p_rule=p_rule, k_block=k_block).float()
    args = (q, k, v) if layout == "BNSD" else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = fp8_attention_forward(*(t.to(cuda) for t in args), layout=layout, recipe=recipe, p_rule=p_rule,
                                k_block=k_block).cpu().float()
    out = out if layout == "BNSD" else out.transpose(1, 2)
    case = (dtype, layout, sq, skv, n, recipe, p_rule, k_block)
    assert bool(torch.isfinite(out).all()), case
    err = (out - want).abs().max().item()
    assert oa.cosine(out, want) >= 0.9999 and err <= 2.0 ** -5 * max(1.0, want.abs().max().item()), (case, err)


@pytest.mark.parametrize("seed", range(16))
def test_varlen_random_sequences(cuda, seed):
    import mindiesd
    from oracle.attention import attention_varlen
    r = random.Random(500 + seed)
    nseq, (n, nkv), causal, d = r.randint(1, 6), _heads(r), r.random() < 0.5, r.choice([128, 128, 64])
    lens_q = [r.choice([0, 1, 7, 64, 100, 129, 300, 513]) for _ in range(nseq)]
    lens_k = [r.choice([1, 5, 64, 77, 128, 200, 257, 640]) for _ in range(nseq)]
    if sum(lens_q) == 0:
        lens_q[0] = 5
    cu_q = torch.tensor([0] + lens_q).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + lens_k).cumsum(0).to(torch.int32)
    q, k, v = (_rnd((sum(lens_q), n, d), seed, torch.bfloat16), _rnd((sum(lens_k), nkv, d), seed + 1, torch.bfloat16),
               _rnd((sum(lens_k), nkv, d), seed + 2, torch.bfloat16))
    on_device = r.random() < 0.5   # the cumulative lengths may live on either side
    out = mindiesd.attention_forward_varlen(q.to(cuda), k.to(cuda), v.to(cuda), cu_q.to(cuda) if on_device else cu_q,
                                            cu_k.to(cuda) if on_device else cu_k, causal=causal).cpu()
    want = attention_varlen(q, k, v, cu_q, cu_k, d ** -0.5, causal)
    assert not torch.isnan(out.float()).any()
    # short sequences: few keys per row, see test_masked_or_causal_random_shape for the bound
    assert (out.float() - want.float()).abs().max().item() <= 5e-2, (lens_q, lens_k, n, nkv, d, causal)


@pytest.mark.parametrize("seed", range(16))
def test_ada_attention_random_mask(cuda, seed):
    import mindiesd  # noqa: F401
    from oracle import ada_bsa as oab
    r = random.Random(600 + seed)
    s, (n, nkv), b = r.choice([130, 256, 500, 769, 1100, 1537]), _heads(r), r.choice([1, 2])
    causal, layout, dtype = r.random() < 0.5, r.choice(["BNSD", "BSND"]), r.choice([torch.bfloat16, torch.float16])
    nb = (s + 127) // 128
    q, k, v = _rnd((b, n, s, 128), seed, dtype), _rnd((b, nkv, s, 128), seed + 1, dtype), _rnd((b, nkv, s, 128), seed + 2, dtype)
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(b, n, nb, nb, generator=g) > r.choice([0.2, 0.5, 0.8])
    if causal:
        m &= torch.ones(nb, nb).tril().bool()
    smask = torch.zeros(b, n, nb, (nb + 31) // 32 * 32, dtype=torch.int8)
    smask[..., :nb] = m.to(torch.int8)
    want = oab.ada_block_sparse_attention(q, k, v, m.numpy(), causal=causal, rules="kernel")
    args = (q, k, v) if layout == "BNSD" else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = torch.ops.mindiesd.ada_block_sparse_attention(
        *(t.to(cuda) for t in args), smask.to(cuda), m.sum(-1).to(torch.int32).to(cuda), input_layout=layout,
        sparse_size=128, num_heads=n, num_key_value_heads=nkv, scale_value=128 ** -0.5, causal=causal).cpu()
    out = out if layout == "BNSD" else out.transpose(1, 2)
    assert not torch.isnan(out.float()).any()
    eb, ok, mx = oa.ref_compare(want, out, 2.0 ** -6)
    assert ok, (eb, mx, b, n, nkv, s, causal, layout, dtype)


@pytest.mark.parametrize("seed", range(16))
def test_mxfp8_gemm_random_shape(cuda, seed):
    """MXFP8 GEMM on random shapes: row counts off the 256-row tiles (1 row up), K any multiple of 128, output widths
    off the tile widths, with and without SwiGLU and bias, both output dtypes; within 2^-7 relative + 1e-3 of the
    oracle's exact product of the dequantised operands (tests/test_gpu_mxfp8_gemm.py's bound)."""
    from mindiesd.layers.quant import mx_quantize, mxfp8_matmul
    from oracle import quant as oq
    r = random.Random(900 + seed)
    m = r.choice([1, 7, 255, 256, 257, 511, 513, r.randrange(1, 1500)])
    k = 128 * r.randrange(1, 13)
    swiglu = r.random() < 0.5
    n = (16 if swiglu else 8) * r.randrange(1, 80)
    out_dtype = r.choice([torch.bfloat16, torch.float16])
    x, w = _rnd((m, k), seed, torch.bfloat16), _rnd((n, k), seed + 1, torch.bfloat16) * 0.05
    bias = _rnd((n,), seed + 2, torch.float32) if r.random() < 0.5 else None
    y = oq.mxfp8_gemm(x, w, bias)
    if swiglu:
        gate, up = y[:, :n // 2], y[:, n // 2:]
        y = gate / (1.0 + torch.exp(-gate)) * up
    xq, xs = mx_quantize(x.to(cuda))
    wq, ws = mx_quantize(w.to(cuda))
    out = mxfp8_matmul(xq, xs, wq, ws, None if bias is None else bias.to(cuda), out_dtype, swiglu=swiglu).cpu()
    assert out.shape == (m, n // 2 if swiglu else n) and out.dtype == out_dtype
    err = (out.double() - y).abs()
    assert bool((err <= 2.0 ** -7 * y.abs() + 1e-3).all()), (err.max().item(), m, k, n, swiglu, bias is not None, out_dtype)
