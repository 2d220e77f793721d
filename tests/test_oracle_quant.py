"""Pins the quantisation oracle against the published formats: OCP FP8 E4M3 (all 256 codes, torch's
own float8_e4m3fn casts, rounding ties, saturation) and OCP MX (power-of-two shared scales, element
range), plus closed-form properties of the block scales and of the dequantised products."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from oracle.attention import attention_math, cosine


def test_e4m3_all_codes_round_trip_and_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    vals = oq.e4m3_decode(codes)
    tv = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    finite = ~np.isnan(tv)
    assert np.isnan(vals[~finite]).all() and (~finite).sum() == 2          # 0x7f and 0xff only
    assert np.array_equal(vals[finite], tv[finite])
    assert vals[0x7e] == 448.0 and vals[0x08] == 2.0 ** -6 and vals[0x01] == 2.0 ** -9
    back = oq.e4m3_encode(vals[finite])
    keep = codes[finite]
    assert np.array_equal(back[keep != 0x80], keep[keep != 0x80])           # -0 encodes as 0x80 too
    assert back[keep == 0x80][0] == 0x80


def test_e4m3_rounding_matches_torch_cast_and_saturates():
    g = torch.Generator().manual_seed(0)
    x = torch.cat([torch.randn(20000, generator=g) * s for s in (1e-3, 0.05, 1.0, 30.0, 200.0)])
    x = x.clamp(-448, 448)
    want = x.to(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(oq.e4m3_round(x.numpy()), want)
    # ties go to the even mantissa: 1.0625 is halfway between 1.0 (even) and 1.125
    assert oq.e4m3_round(np.float32([1.0625, 1.1875, 2.0 ** -10, 3 * 2.0 ** -10])).tolist() == [1.0, 1.25, 0.0, 2 ** -8]
    # saturation (torch's cast gives NaN above the range; the oracle and the kernels clamp)
    assert oq.e4m3_round(np.float32([460, 480, 1e6, -1e6])).tolist() == [448.0, 448.0, 448.0, -448.0]


def test_block_quant_scales_and_error_bound():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 300, 128, generator=g).to(torch.bfloat16)
    x[1, 128:256] = 0                                   # an all-zero block
    codes, scale = oq.dynamic_block_quant(x, 128, 128)
    assert codes.shape == x.shape and scale.shape == (3, 3, 1) and scale.dtype == torch.float32
    amax = torch.stack([x[:, i * 128:(i + 1) * 128].float().abs().amax(dim=(1, 2)) for i in range(3)], 1)
    assert torch.equal(scale[..., 0][amax > 0], (amax / 448.0)[amax > 0]) and scale[1, 1, 0] == 1.0
    deq = oq.dequant_block(codes, scale, 128, 128)
    # E4M3 keeps 4 significant bits: relative error <= 2^-4 for normals, absolute <= scale * 2^-10 below
    err = (deq - x.float()).abs()
    bound = torch.maximum(x.float().abs() * 2.0 ** -4, scale.repeat_interleave(128, 1)[:, :300] * 2.0 ** -10)
    assert (err <= bound + 1e-12).all()
    assert (oq.e4m3_decode(codes.numpy()).__abs__().max() == 448.0)   # the block maximum maps to the largest code
    c256, s256 = oq.dynamic_block_quant(x, 256, 128)
    assert s256.shape == (3, 2, 1)


def test_per_channel_quant():
    g = torch.Generator().manual_seed(2)
    v = torch.randn(2, 500, 128, generator=g) * torch.linspace(0.1, 5, 128)
    codes, sc = oq.per_channel_quant(v)
    assert sc.shape == (2, 128) and torch.allclose(sc, v.abs().amax(dim=1) / 448.0)
    deq = torch.from_numpy(oq.e4m3_decode(codes.numpy())) * sc[:, None, :]
    assert ((deq - v).abs() <= v.abs() * 2.0 ** -4 + sc[:, None, :] * 2.0 ** -10).all()


def test_mx_quant_follows_ocp_mx():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 256, generator=g) * torch.logspace(-3, 3, 64)[:, None]
    x[5, 32:64] = 0
    codes, e8 = oq.mx_quant(x)
    assert codes.shape == (64, 256) and e8.shape == (64, 8) and e8.dtype == torch.uint8
    amax = x.reshape(64, 8, 32).abs().amax(-1)
    expect = torch.floor(torch.log2(amax.double().clamp(min=1e-300))) - 8 + 127
    assert torch.equal(e8.double()[amax > 0], expect[amax > 0]) and e8[5, 1] == 0
    # the scaled block maximum lies in [256, 512): the top of the E4M3 range, saturated at 448
    q = torch.from_numpy(oq.e4m3_decode(codes.numpy())).reshape(64, 8, 32).abs().amax(-1)
    assert ((q >= 256) & (q <= 448))[amax > 0].all()
    deq = oq.mx_dequant(codes, e8)
    rel = ((deq - x.double()).abs() / amax.repeat_interleave(32, 1).clamp(min=1e-30)).max()
    assert rel <= 0.125 + 1e-9        # saturation of [448, 512) costs at most 12.5 % of the block maximum
    # torch's float8_e8m0fnu agrees on what the scale bytes mean
    assert torch.equal(e8.view(torch.float8_e8m0fnu).float()[amax > 0],
                       torch.exp2(e8.float() - 127)[amax > 0])


def test_mxfp8_gemm_swiglu_close_to_unquantised():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(96, 512, generator=g)
    w = torch.randn(2 * 80, 512, generator=g) * 0.02
    got = oq.mxfp8_gemm_swiglu(x, w, torch.float32)
    y = x.double() @ w.double().t()
    want = torch.nn.functional.silu(y[:, :80]) * y[:, 80:]
    cos = float((got.double().flatten() @ want.flatten()) / (got.double().norm() * want.norm()))
    assert got.shape == (96, 80) and cos > 0.995
    # linearity in the power-of-two scale: scaling x by 4 scales the GEMM by exactly 4
    assert torch.equal(oq.mxfp8_gemm(x * 4, w), oq.mxfp8_gemm(x, w) * 4)


def test_fp8_attention_close_to_unquantised():
    from oracle.attention import attention_fp64, cosine
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 2, 300, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    out = oq.fp8_attention(q, k, v)
    assert out.dtype == torch.bfloat16
    for n in range(2):
        assert cosine(out[0, n], attention_fp64(q[0, n], k[0, n], v[0, n], 128 ** -0.5)) > 0.995


# ---- power-of-two block scales (recipe of the log2-domain FP8 attention kernel; not in the reference) -------------
def test_pow2_ceil_closed_forms():
    sc = np.array([1.0, 1.0000001, 0.75, 0.5, 0.50000006, 3.0, 4.0, 2.0 ** -20, 1e-45], dtype=np.float32)
    want = np.array([1.0, 2.0, 1.0, 0.5, 1.0, 4.0, 4.0, 2.0 ** -20, 2.0 ** -126], dtype=np.float32)
    assert np.array_equal(oq.pow2_ceil(sc), want)


def test_pow2_block_quant_properties():
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(2, 300, 128, generator=g) * 3).to(torch.bfloat16)
    x[0, :128] = 0
    codes, scale = oq.dynamic_block_quant(x, 128, 128, pow2=True)
    _, plain = oq.dynamic_block_quant(x, 128, 128)
    s, p = scale.numpy(), plain.numpy()
    nz = p != 1.0
    assert (np.frexp(s)[0] == 0.5).all()                       # powers of two
    assert (s[nz] >= p[nz]).all() and (s[nz] < 2 * p[nz]).all()  # smallest one not below amax / 448
    assert s[0, 0, 0] == 1.0 and (codes[0, :128].numpy() & 0x7f == 0).all()
    deq = oq.dequant_block(codes, scale, 128, 128)
    rel = (deq - x.float()).abs() / x.float().abs().clamp_min(1e-3)
    big = x.float().abs() > 0.05 * x.float().abs().amax(dim=(-1, -2), keepdim=True)
    assert rel[big].max() <= 2.0 ** -4 + 1e-6                  # E4M3: 3 mantissa bits, half an ulp
    assert int(codes.max()) <= 0x7e | 0x80 and (codes.numpy() & 0x7f).max() <= 0x7e  # never NaN / beyond 448


def test_prescale_by_a_power_of_two_only_moves_the_scale():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(1, 256, 128, generator=g).to(torch.bfloat16)
    c1, s1 = oq.dynamic_block_quant(x, 128, 128, 1.0, True)
    c2, s2 = oq.dynamic_block_quant(x, 128, 128, 0.125, True)
    assert torch.equal(c1, c2) and torch.equal(s2, s1 * 0.125)


def test_fp8_attention_recipes_agree_with_each_other_and_with_plain_attention():
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, 2, 384, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    a, b = oq.fp8_attention(q, k, v), oq.fp8_attention(q, k, v, pow2=True)
    ref = attention_math(q, k, v, None, 128 ** -0.5, head_first=True)
    assert cosine(a, b) > 0.997 and cosine(b, ref) > 0.995 and cosine(a, ref) > 0.995


def test_linear_code_rule_closed_forms():
    """The linear rule writes the E4M3 code 8 (x + 7) + 118 - 56: integers x give exact powers of two, the value read
    back from the code is 2^floor(x') (1 + frac(x')) with the fraction rounded to eighths, never more than 6.2 % above
    and (by the rounding) 3.2 % below 2^x' down to the smallest normal, and the code saturates instead of wrapping."""
    x = np.arange(-13, 2, dtype=np.float32)                       # x' = x + 7.75 in [-5.25, 8.75]
    y = np.float32(8.0) * x + oq.L_SEED
    vals = oq.e4m3_decode(oq.linear_p_codes(y)).astype(np.float64)
    assert np.array_equal(oq.linear_p_codes(y), (8 * (x + 14.75)).astype(np.uint8))
    assert np.allclose(vals, np.exp2(np.floor(x + 7.75)) * 1.75)  # frac(x') = 0.75 -> mantissa 6/8
    rng = np.random.default_rng(0)
    xr = rng.uniform(-13.5, 1.0, 100000).astype(np.float32)
    v = oq.e4m3_decode(oq.linear_p_codes(np.float32(8.0) * xr + oq.L_SEED)).astype(np.float64)
    ratio = v / np.exp2(xr.astype(np.float64) + 7.75)
    assert ratio.max() <= 1.062 * (1 + 2.0 ** -4) and ratio.min() >= 1 - 2.0 ** -4
    assert abs(ratio.mean() - 1.04) < 0.005 and ratio.std() < 0.035
    # largest code the kernel can reach: score = reference + threshold -> 126 (= 448), never the NaN code 127
    assert oq.linear_p_codes(np.float32(8.0) * oq.L_TAU + oq.L_SEED) == 126
    assert np.array_equal(oq.linear_p_codes(np.array([-1e9, -np.inf, np.nan, 0.49, 0.5, 1.5, 2.5, 1e9], np.float32)),
                          np.array([0, 0, 0, 0, 0, 2, 2, 255], np.uint8))


@pytest.mark.parametrize("p_rule", ["linear", "exp2"])
@pytest.mark.parametrize("pow2", [False, True])
def test_requantised_probabilities_stay_within_a_bound_of_the_plain_form(pow2, p_rule):
    """``fp8_attention(requant_p=True)`` (P rounded to E4M3 per 128-key tile, denominator from the rounded values,
    lazily moved reference) against the plain quantise -> dequantise form: an E4M3 probability carries at most
    2^-4 relative error, and the errors of a row average out over its keys - the outputs differ by far less than
    2^-5 of the largest value, a factor on P that did not cancel or a missed rescale would not."""
    import torch
    g = torch.Generator().manual_seed(3)
    def make():
        x = torch.randn(1, 2, 700, 128, generator=g)
        return torch.where(torch.rand(1, 2, 700, 128, generator=g) < 0.01, x * 8, x).to(torch.bfloat16)
    q, k, v = make(), make(), make()
    k[:, :, 300:] *= 1.5            # rising row maxima: the reference has to move after the first tile
    a = oq.fp8_attention(q, k, v, pow2=pow2).float()
    b = oq.fp8_attention(q, k, v, pow2=pow2, requant_p=True, p_rule=p_rule).float()
    assert torch.nn.functional.cosine_similarity(a.flatten(), b.flatten(), dim=0) >= 0.9999
    assert (a - b).abs().max() <= 2.0 ** -5 * v.float().abs().max()
    # one key tile, uniform scores: every probability is the same power of two, the rounding is exact and the
    # result is the mean of the (de)quantised values whatever the recipe does with the reference
    kz = torch.zeros(1, 1, 100, 128, dtype=torch.bfloat16)
    vz = make()[:, :1, :100]
    out = oq.fp8_attention(q[:, :1, :40], kz, vz, pow2=pow2, requant_p=True, p_rule=p_rule).float()
    codes, sc = oq.per_channel_quant(vz)
    mean = (torch.from_numpy(oq.e4m3_decode(codes.numpy())) * sc[..., None, :]).mean(dim=-2, keepdim=True)
    assert (out - mean.to(torch.bfloat16).float()).abs().max() <= 2.0 ** -7 * mean.abs().max()
