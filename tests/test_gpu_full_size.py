"""The three large workloads at their full sizes on the GPU (block-sparse pipeline at B1 N40 S75600, FP8
attention at B1 N40 S32760, MXFP8 GEMM + SwiGLU at M32760 K5120 N2x13824): the CPU oracle checks samples
(whole heads of the mask, whole query blocks / rows of the outputs) and size-independent properties
(forced blocks, list/mask consistency, scale closed forms, power-of-two linearity) cover the rest."""
import math

import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import quant as oq
from oracle import rainfusion as orf
from workloads import dense_inputs, smooth_field_inputs

pytestmark = pytest.mark.gpu


def _gpu_randn(shape, seed, device, mul=1.0):
    g = torch.Generator(device=device).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=device) * mul).to(torch.bfloat16)


def test_dense_wan14b_720p_row_samples(cuda):
    """The benchmarked launch itself (B1 N40 S75600 D128, the benchmark's seeded inputs): first, middle and tail
    query tiles of two heads against the oracle's attention_math, max-abs <= 2e-2 and cosine >= 0.9999."""
    import mindiesd
    cfg = dict(B=1, N=40, S=75600, D=128)
    q, k, v = dense_inputs(cfg, cuda, seed=1)
    out = mindiesd.attention_forward(q, k, v, head_first=True)
    assert out.shape == q.shape and bool(torch.isfinite(out[:, ::13].float()).all())
    s = cfg["S"]
    for head in (0, 39):
        qh, kh, vh = (t[:, head:head + 1].cpu() for t in (q, k, v))
        for rows in (slice(0, 256), slice(37760, 38016), slice(s - 336, s)):   # the last: tiles 294 (whole) and 295 (80 rows)
            ref = oa.attention_math_rows(qh, kh, vh, 128 ** -0.5, row_chunk=256, q_rows=rows)
            got = out[:, head:head + 1, rows].cpu()
            err = (got.float() - ref.float()).abs().max().item()
            assert err <= 2e-2 and oa.cosine(got, ref) >= 0.9999, (head, rows, err, oa.cosine(got, ref))


def test_sparse_pipeline_wan14b_720p(cuda):
    from mindiesd.layers.flash_attn import rainfusion as rf
    grid, n, d = (21, 45, 80), 40, 128
    s = grid[0] * grid[1] * grid[2]
    nb = math.ceil(s / 128)
    # the block-sparse workload's own inputs: Gaussian-filtered (sigma 2 tokens) spatio-temporal field + 0.3 N(0,1)
    q, k, v = smooth_field_inputs(dict(B=1, N=n, S=s, D=d, grid=grid), cuda, seed=3)
    out, mask = rf.bsa_sparse_attention_v3(q, k, v, grid, sparsity=0.75, input_layout="BNSD", keep_diagonal=True)
    assert out.shape == q.shape and mask.shape == (1, n, nb, nb) and mask.dtype == torch.int8
    # ---- mask properties over all heads --------------------------------------------------------------------------
    keep_len = orf.keep_len_of(nb, 0.75)
    cnt = mask.sum(dim=-1, dtype=torch.int32)
    assert int(cnt.min()) >= keep_len
    forced = orf.apply_forced_blocks(torch.zeros(1, 1, nb, nb, dtype=torch.bool), 0, 128, grid, True)[0, 0]
    assert forced.any() and bool(mask[0, :, forced.to(cuda)].all()), "first-frame blocks must be kept"
    dg = torch.arange(nb, device=cuda)
    assert bool(mask[0, :, dg, dg].all())
    idx, cnt2 = rf.mask_to_lists(mask)
    assert torch.equal(cnt2.reshape(cnt.shape), cnt)
    row = idx[0, 7, 300, : int(cnt[0, 7, 300])].cpu()
    assert torch.equal(row, torch.nonzero(mask[0, 7, 300].cpu()).flatten().to(row.dtype))
    density = float(cnt.sum()) / (n * nb * nb)
    assert 0.25 <= density <= 0.40, density
    # ---- pooled means and masks of two heads against the oracle: bit-exact ------------------------------------
    heads = [3, 38]
    order = torch.from_numpy(np.asarray(orf.window_order(*grid)).astype(np.int64))
    qh, kh, vh = (t[:, heads].cpu() for t in (q, k, v))
    q_, k_, v_, pool = orf.do_tensor_rearrange_pooling(qh, kh, vh, 0, 128, grid, grid, "BNSD")
    assert torch.equal(q_[0, 0], qh[0, 0][order])
    want_mask = orf.get_blockwise_mask(pool, 0, 0.75, d ** -0.5, 128, grid, grid, "BNSD", return_binary=True,
                                       keep_diagonal=True)
    assert torch.equal(mask[:, heads].cpu(), want_mask), "block mask must be bit-exact"
    # ---- three query blocks of one head against the oracle (first-frame block, a middle one, the tail block) ----
    blocks = [0, 311, nb - 1]
    rows = torch.cat([torch.arange(b * 128, min((b + 1) * 128, s)) for b in blocks])
    sub_mask = want_mask[:, :1, blocks]
    pad = 128 * len(blocks) - rows.numel()  # the tail block is short: pad with copies of its last row
    rows_p = torch.cat([rows, rows[-1:].expand(pad)])
    ref = oa.block_sparse_attention(q_[:, :1, rows_p], k_[:, :1], v_[:, :1], sub_mask)[:, :, : rows.numel()]
    got = out[0, heads[0]].cpu()[order[rows]]
    eb, ok, mx = oa.ref_compare(ref[0, 0], got, 2.0 ** -6)
    assert ok, (eb, mx)


def test_fp8_attention_wan14b_480p(cuda):
    from mindiesd.layers.quant import fa_block_quant_preprocess, fp8_attention_forward
    n, s, d = 40, 32760, 128
    g = torch.Generator(device=cuda).manual_seed(5)

    def make():
        x = torch.randn((1, n, s, d), generator=g, device=cuda)
        m = torch.rand((1, n, s, d), generator=g, device=cuda) < 0.01
        return torch.where(m, x * 8, x).to(torch.bfloat16)

    q, k, v = make(), make(), make()
    out = fp8_attention_forward(q, k, v, layout="BNSD")
    assert out.shape == q.shape and out.dtype == torch.bfloat16 and bool(torch.isfinite(out.float()).all())
    # quantisation at full size: scale = amax / 448 per (head, 128 tokens), reconstruction within half an E4M3 step
    codes, scale = fa_block_quant_preprocess(k, block_size=128, layout="BNSD")
    nblk = math.ceil(s / 128)
    pad = nblk * 128 - s
    kp = torch.nn.functional.pad(k.float(), (0, 0, 0, pad))
    amax = kp.reshape(1, n, nblk, 128 * d).abs().amax(dim=-1)
    # the division is done on the CPU: IEEE division there, whereas the GPU's torch division need not round correctly
    assert torch.equal(scale.reshape(1, n, nblk).cpu(), amax.cpu() / 448.0)
    deq = codes.float() * scale.reshape(1, n, nblk, 1).repeat_interleave(128, dim=2)[:, :, :s]
    step = torch.maximum(k.float().abs() * 2.0 ** -4, scale.reshape(1, n, nblk, 1).repeat_interleave(128, dim=2)[:, :, :s] * 2.0 ** -10)
    assert bool(((deq - k.float()).abs() <= step * 1.0001).all())
    del kp, deq, step, codes
    # two query blocks of two heads against the quantise -> dequantise oracle (cosine >= 0.999)
    # (each recipe against the oracle of the same recipe)
    out_p2 = fp8_attention_forward(q, k, v, layout="BNSD", recipe="pow2")
    out_ex = fp8_attention_forward(q, k, v, layout="BNSD", p_rule="exp2")
    for head in (0, 39):
        qs = q[:, head:head + 1, 128 * 100: 128 * 102].cpu()
        for res, p2, rule in ((out, False, "linear"), (out_p2, True, "linear"), (out_ex, False, "exp2")):
            want = oq.fp8_attention(qs, k[:, head:head + 1].cpu(), v[:, head:head + 1].cpu(), pow2=p2)
            got = res[:, head:head + 1, 128 * 100: 128 * 102].cpu()
            assert oa.cosine(got, want) >= 0.999, (p2, oa.cosine(got, want))
            # and tightly against the oracle that re-quantises P per tile the way the kernel does
            mirror = oq.fp8_attention(qs, k[:, head:head + 1].cpu(), v[:, head:head + 1].cpu(), pow2=p2, requant_p=True,
                                      p_rule=rule)
            assert oa.cosine(got, mirror) >= 0.99998, (p2, oa.cosine(got, mirror), oa.cosine(got, want))
            print(f"fp8 full size head {head} pow2 {p2} {rule}: cosine vs plain oracle {oa.cosine(got, want):.7f}, vs P-requantising oracle {oa.cosine(got, mirror):.7f}", flush=True)


def test_mxfp8_gemm_swiglu_ffn_shape(cuda):
    from mindiesd.layers.quant import mx_quantize, mxfp8_matmul
    m, kdim, f = 32760, 5120, 13824
    x = _gpu_randn((m, kdim), 7, cuda)
    w = _gpu_randn((2 * f, kdim), 8, cuda, 0.02)
    xq, xs = mx_quantize(x)
    wq, ws = mx_quantize(w)
    out = mxfp8_matmul(xq, xs, wq, ws, None, torch.bfloat16, swiglu=True)
    assert out.shape == (m, f) and bool(torch.isfinite(out.float()).all())
    # row samples (first rows, rows across a tile boundary, the short last tile) x a column sample incl. the last columns
    rows = torch.cat([torch.arange(0, 40), torch.arange(16380, 16400), torch.arange(m - 40, m)])
    cols = torch.cat([torch.arange(0, 96), torch.arange(6900, 6996), torch.arange(f - 64, f)])
    wsub = torch.cat([w[cols.to(cuda)], w[(f + cols).to(cuda)]]).cpu()
    want = oq.mxfp8_gemm_swiglu(x[rows.to(cuda)].cpu(), wsub, torch.float32)
    got = out[rows.to(cuda)][:, cols.to(cuda)].cpu()
    assert oa.cosine(got, want) >= 0.999
    assert bool(((got.float() - want).abs() <= 2.0 ** -7 * want.abs() + 1e-3).all())
    # power-of-two linearity of the plain GEMM: scaling X by 4 moves only the E8M0 exponents
    plain = mxfp8_matmul(xq, xs, wq, ws, None, torch.bfloat16, swiglu=False)
    xq4, xs4 = mx_quantize((x.float() * 4).to(torch.bfloat16))
    assert torch.equal(xq4.view(torch.uint8), xq.view(torch.uint8))
    plain4 = mxfp8_matmul(xq4, xs4, wq, ws, None, torch.bfloat16, swiglu=False)
    assert torch.equal(plain4, (plain.float() * 4).to(torch.bfloat16))
