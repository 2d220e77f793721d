"""Oracle: FP8 / MXFP8 quantisation, FP8 attention and the MXFP8 GEMM+SwiGLU on the CPU
(test infrastructure only).

PARITY UNPINNED against the reference: the reference hands these steps to closed vendor ops
(``torch_npu.npu_dynamic_block_quant`` mindiesd/layers/quant/block_quant.py:43-46,
``npu_fused_infer_attention_score_v2`` mindiesd/quantization/layer.py:304-316,
``npu_dynamic_mx_quant`` / ``npu_quant_matmul`` layer.py:338-361) and mocks them in its own tests
(tests/quantization/test_layer.py:40-54), so there is no reference arithmetic to compare with.
The functions below follow the published formats instead and are pinned against those:

* OCP FP8 E4M3 ("e4m3fn": bias 7, 3 mantissa bits, max 448, no infinities), round to nearest even,
  saturating -- ``e4m3_round`` is a bit-level implementation checked against all 256 codes and
  against torch's ``float8_e4m3fn`` casts.
* block scaling: ``scale = amax / 448`` in fp32 per block, ``q = e4m3(x / scale)`` (an all-zero
  block gets scale 1), dequantisation ``x ~ q * scale``.
* OCP Microscaling (MX) v1.0, MXFP8 E4M3: blocks of 32 along K share an E8M0 scale
  ``2^(floor(log2(amax)) - 8)`` (8 = exponent of the largest E4M3 normal), elements are
  ``e4m3(x / scale)`` saturated to +-448.
"""
import math

import numpy as np
import torch

E4M3_MAX = 448.0


# ---- E4M3 ---------------------------------------------------------------------------------------------
def e4m3_decode(codes):
    """uint8 codes -> float32 (0x7f / 0xff are NaN)."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    sign = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 0x7
    val = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e.astype(np.float64) - 7))
    val = np.where((e == 15) & (m == 7), np.nan, val)
    return (sign * val).astype(np.float32)


def e4m3_encode(x):
    """float32 -> nearest E4M3 code, ties to even, magnitudes above 448 saturate to +-448."""
    x = np.asarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x).astype(np.float64), E4M3_MAX)
    # exponent of the grid: normals have 3 mantissa bits, subnormals a fixed step of 2^-9
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -6)))
    step = np.exp2(e - 3)
    q = np.rint(a / step) * step          # np.rint rounds half to even
    q = np.minimum(q, E4M3_MAX)
    e2 = np.floor(np.log2(np.maximum(q, 2.0 ** -6)))
    mant = np.where(q < 2.0 ** -6, q / 2.0 ** -9, (q / np.exp2(e2) - 1.0) * 8.0)
    expo = np.where(q < 2.0 ** -6, 0, e2 + 7)
    code = (expo.astype(np.int32) << 3) | np.rint(mant).astype(np.int32)
    code = np.where(np.signbit(x), code | 0x80, code)
    return code.astype(np.uint8)


def e4m3_round(x):
    """float32 -> float32 value of the nearest E4M3 number (RNE, saturating)."""
    return e4m3_decode(e4m3_encode(x))


# ---- block quantisation of attention operands ----------------------------------------------------------
def pow2_ceil(sc):
    """Smallest power of two >= sc (fp32 array of positive normal numbers; at least 2^-126)."""
    m, e = np.frexp(sc.astype(np.float32))          # sc = m * 2^e, m in [0.5, 1)
    e = np.where(m == 0.5, e - 1, e)
    return np.ldexp(np.float32(1.0), np.maximum(e, -126)).astype(np.float32)


def dynamic_block_quant(x, row_block=128, col_block=128, prescale=1.0, pow2=False):
    """[..., S, D] -> (codes uint8 same shape, scale fp32 [..., ceil(S/row_block), ceil(D/col_block)]).
    One scale per (row_block tokens x col_block channels) tile: scale = amax/448, q = e4m3(x/scale).
    ``prescale`` multiplies x first (one fp32 rounding); ``pow2`` rounds the scale up to a power of two - the
    recipe of the log2-domain FP8 attention kernel (not in the reference)."""
    xf = (x.float().numpy() * np.float32(prescale)).astype(np.float32)
    s, d = xf.shape[-2:]
    nb_r, nb_c = math.ceil(s / row_block), math.ceil(d / col_block)
    codes = np.zeros(xf.shape, dtype=np.uint8)
    scale = np.ones(xf.shape[:-2] + (nb_r, nb_c), dtype=np.float32)
    for i in range(nb_r):
        for j in range(nb_c):
            rs, cs = slice(i * row_block, (i + 1) * row_block), slice(j * col_block, (j + 1) * col_block)
            blk = xf[..., rs, cs]
            amax = np.abs(blk).max(axis=(-1, -2)).astype(np.float32)
            sc = np.where(amax > 0, amax / np.float32(E4M3_MAX), np.float32(1.0)).astype(np.float32)
            if pow2:
                sc = np.where(amax > 0, pow2_ceil(sc), np.float32(1.0)).astype(np.float32)
            scale[..., i, j] = sc
            codes[..., rs, cs] = e4m3_encode(blk / sc[..., None, None])
    return torch.from_numpy(codes), torch.from_numpy(scale)


def rot_block_quant(x, rot, row_block=128, prescale=1.0, pow2=False):
    """FP8RotateQuantFA's first two steps (mindiesd/quantization/layer.py:284-296) on the CPU:
    ``torch.matmul(x, rot)`` in the 16-bit input type (fp32 accumulation, one rounding), then
    ``dynamic_block_quant`` over (row_block tokens x all channels)."""
    y = torch.matmul(x.float(), rot.to(x.dtype).float()).to(x.dtype)
    return dynamic_block_quant(y, row_block, x.shape[-1], prescale, pow2)


def dequant_block(codes, scale, row_block=128, col_block=128):
    q = torch.from_numpy(e4m3_decode(codes.numpy()))
    s, d = q.shape[-2:]
    sc = scale.repeat_interleave(row_block, dim=-2)[..., :s, :].repeat_interleave(col_block, dim=-1)[..., :d]
    return q * sc


def per_channel_quant(v):
    """[..., S, D] -> (codes, scale [..., D]): one scale per channel over the whole sequence."""
    vf = v.float().numpy()
    amax = np.abs(vf).max(axis=-2).astype(np.float32)
    sc = np.where(amax > 0, amax / np.float32(E4M3_MAX), np.float32(1.0)).astype(np.float32)
    return torch.from_numpy(e4m3_encode(vf / sc[..., None, :])), torch.from_numpy(sc)


def fp8_attention(query, key, value, scale=None, pow2=False, requant_p=False, p_rule="linear", k_block=128):
    """FP8 attention of the Wan2.1-14B 480p workload, BNSD: Q and K quantised per (head, 128-token
    block) over all channels, V per (head, channel); bf16-typed output.
    ``requant_p=False``: the quantise -> dequantise path - everything is dequantised and run through plain
    softmax(scale QK^T)V in fp32.
    ``requant_p=True``: additionally the workload's "P re-quantised to e4m3 per tile", with the choices of the GPU
    kernel: keys in tiles of 128; per tile P = 2^4 * exp2(score - reference) rounded to E4M3 (ties to even), where
    the reference is a running maximum per query row that is only moved when, in the row's group of 32 consecutive
    query rows, some row's tile maximum exceeds its reference by more than 2^4 (so P <= 256 < 448); the
    denominator is the sum of the ROUNDED probabilities, the numerator their product with the V codes; both are
    rescaled by 2^(old - new reference) when the reference moves.  That is ``p_rule="exp2"``.
    ``p_rule="linear"`` (the kernel's default): the E4M3 CODE of a probability is computed directly,
    code = rne(8 * (score - reference) + 8 * (7.75 + 7)) saturated to [0, 255] - read back as E4M3 that is
    2^floor(x') * (1 + frac(x')) with frac rounded to eighths, x' = score - reference + 7.75: the exponential with
    its mantissa interpolated linearly between powers of two (code 8 e + m stands for 2^(e-7) (1 + m/8)); the reference
    moves when a row of the group exceeds it by more than 2^1 (so the code stays <= 126 = 448).
    ``k_block``: tokens per K scale (128; 256 = the K recipe of the reference's FP8RotateQuantFA, layer.py:297-302)."""
    d = query.shape[-1]
    if scale is None:
        scale = d ** -0.5
    if pow2:
        # log2-domain recipe: the query carries scale * log2(e), block scales are powers of two; the dequantised
        # scores are then in log2 units, i.e. ln(2) stands where the softmax scale stood
        qc, qs = dynamic_block_quant(query, 128, d, scale * 1.4426950408889634, True)
        kc, ks = dynamic_block_quant(key, k_block, d, 1.0, True)
        scale = math.log(2.0)
    else:
        qc, qs = dynamic_block_quant(query, 128, d)
        kc, ks = dynamic_block_quant(key, k_block, d)
    vc, vs = per_channel_quant(value)
    if requant_p:
        return _fp8_attention_requant(qc, qs, kc, ks, vc, vs, np.float32(scale * 1.4426950408889634), pow2,
                                      p_rule, k_block).to(query.dtype)
    qd, kd = dequant_block(qc, qs, 128, d), dequant_block(kc, ks, k_block, d)
    vd = torch.from_numpy(e4m3_decode(vc.numpy())) * vs[..., None, :]
    out = torch.empty(query.shape, dtype=torch.float32)
    for r0 in range(0, query.shape[-2], 2048):
        s = (qd[..., r0:r0 + 2048, :] @ kd.transpose(-1, -2)) * scale
        out[..., r0:r0 + 2048, :] = torch.softmax(s, dim=-1) @ vd
    return out.to(query.dtype)


P_SHIFT, P_TAU, ROW_GROUP, KEY_TILE = np.float32(4.0), np.float32(4.0), 32, 128
L_SHIFT, L_TAU = np.float32(7.75), np.float32(1.0)       # the linear code rule
L_SEED = np.float32(8.0) * (L_SHIFT + np.float32(7.0))   # the code of score == reference (118)


def linear_p_codes(y):
    """E4M3 codes of the linear rule from y = 8 * (score - reference) + 118 (fp32): rne(y) saturated to [0, 255]
    (what v_cvt_pk_u8_f32 does: ties to even, negative and NaN -> 0)."""
    y = np.nan_to_num(np.asarray(y, np.float32), nan=0.0, posinf=255.0, neginf=0.0)
    return np.clip(np.rint(y), 0, 255).astype(np.uint8)


def _fp8_attention_requant(qc, qs, kc, ks, vc, vs, scale_log2, pow2, p_rule="linear", k_block=128):
    """The tile loop behind ``fp8_attention(requant_p=True)`` on the quantised operands (codes + scales)."""
    linear = p_rule == "linear"
    tau = L_TAU if linear else P_TAU
    q8, k8, v8 = e4m3_decode(qc.numpy()), e4m3_decode(kc.numpy()), e4m3_decode(vc.numpy())
    qsn, ksn, vsn = qs.numpy()[..., 0], ks.numpy()[..., 0], vs.numpy()
    b, n, sq, d = q8.shape
    skv = k8.shape[2]
    out = np.zeros((b, n, sq, d), dtype=np.float32)
    for bi in range(b):
        for ni in range(n):
            for r0 in range(0, sq, ROW_GROUP):
                r1 = min(r0 + ROW_GROUP, sq)
                rows = r1 - r0
                qsc = qsn[bi, ni, r0 // 128]
                m_run = np.full(rows, 0.0 if pow2 else -np.inf, dtype=np.float32)
                l_run = np.zeros(rows, dtype=np.float32)
                o_run = np.zeros((rows, d), dtype=np.float32)
                first = True
                for t0 in range(0, skv, KEY_TILE):
                    t1 = min(t0 + KEY_TILE, skv)
                    raw = q8[bi, ni, r0:r1] @ k8[bi, ni, t0:t1].T                     # exact sums of code products
                    if pow2:  # the scales are powers of two (applied by the matrix instruction's exponents)
                        s = (raw * (qsc * ksn[bi, ni, t0 // k_block])).astype(np.float32)
                        mx = s.max(axis=1) - m_run
                        if first or (mx > tau).any():
                            delta = mx if first else np.maximum(mx, np.float32(0))
                            # (first tile: sums and outputs are still zero, the factor is 1; 2^-delta may overflow)
                            alpha = np.ones_like(delta) if first else np.exp2(-delta).astype(np.float32)
                            m_run = m_run + delta
                            l_run *= alpha
                            o_run *= alpha[:, None]
                    else:     # amax/448 scales folded into the softmax scale of the tile
                        c = np.float32(np.float32(qsc * scale_log2) * ksn[bi, ni, t0 // k_block])
                        s = (raw * c).astype(np.float32)
                        mx = s.max(axis=1)
                        if (mx > m_run + tau).any():
                            m_new = np.maximum(m_run, mx)
                            alpha = np.where(np.isinf(m_run), np.float32(0), np.exp2(m_run - m_new)).astype(np.float32)
                            m_run = m_new
                            l_run *= alpha
                            o_run *= alpha[:, None]
                    first = False
                    if linear:
                        # one multiply-add per score on the GPU: (8 c) raw + (118 - 8 reference), rounded once
                        off8 = (np.float64(L_SEED) - 8.0 * m_run.astype(np.float64)).astype(np.float32)
                        if pow2:  # the matrix instruction applies 8 x the two scales and starts from off8
                            y = 8.0 * s.astype(np.float64) + off8[:, None]
                        else:
                            y = raw.astype(np.float64) * np.float64(np.float32(c * np.float32(8.0))) + off8[:, None]
                        p8 = e4m3_decode(linear_p_codes(y.astype(np.float32)))
                    else:
                        p8 = e4m3_round(np.exp2(s - (m_run - P_SHIFT)[:, None]).astype(np.float32))
                    l_run += p8.sum(axis=1, dtype=np.float32)
                    o_run += p8 @ v8[bi, ni, t0:t1]
                inv = np.where(l_run > 0, np.float32(1) / np.maximum(l_run, np.float32(1e-30)), np.float32(0))
                out[bi, ni, r0:r1] = o_run * inv[:, None] * vsn[bi, ni][None, :]
    return torch.from_numpy(out)


# ---- MX (microscaling) ----------------------------------------------------------------------------------
def mx_quant(x, block=32):
    """[M, K] -> (codes uint8 [M, K], e8m0 uint8 [M, K/block]); K must be a multiple of ``block``."""
    xf = x.float().numpy()
    m, k = xf.shape
    assert k % block == 0
    blk = xf.reshape(m, k // block, block)
    amax = np.abs(blk).max(axis=-1)
    _, ex = np.frexp(amax)                      # amax = f * 2^ex with f in [0.5, 1)  ->  floor(log2) = ex - 1
    shared = np.where(amax > 0, ex - 1 - 8, -127)
    shared = np.clip(shared, -127, 127).astype(np.int32)
    codes = e4m3_encode(blk / np.exp2(shared.astype(np.float64))[..., None].astype(np.float32)).reshape(m, k)
    return torch.from_numpy(codes), torch.from_numpy((shared + 127).astype(np.uint8))


def mx_dequant(codes, e8m0, block=32):
    q = e4m3_decode(codes.numpy()).astype(np.float64)
    sc = np.exp2(e8m0.numpy().astype(np.float64) - 127)
    return torch.from_numpy(q * np.repeat(sc, block, axis=-1))


def mxfp8_gemm(x, w, bias=None):
    """x [M, K], w [N, K] (both any float dtype) -> fp64 [M, N]: MX-quantise both along K,
    dequantise, multiply exactly."""
    xd = mx_dequant(*mx_quant(x))
    wd = mx_dequant(*mx_quant(w))
    out = xd @ wd.t()
    return out if bias is None else out + bias.double()


def mxfp8_gemm_swiglu(x, w, out_dtype=torch.bfloat16):
    """w = [gate rows | up rows] ([2F, K]); returns silu(x w_gate^T) * (x w_up^T) as ``out_dtype`` [M, F]."""
    y = mxfp8_gemm(x, w)
    f = w.shape[0] // 2
    gate, up = y[:, :f], y[:, f:]
    return (gate / (1.0 + torch.exp(-gate)) * up).to(out_dtype)
