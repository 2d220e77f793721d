"""GPU parity of the FP8 path vs the CPU oracle: quantised codes and scales bit-exact against the
format definition (OCP E4M3, scale = amax/448), attention output cosine >= 0.999 against the
quantise -> dequantise oracle (the stated tolerance of the FP8 workload)."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from oracle.attention import cosine

pytestmark = pytest.mark.gpu


def _outlier_inputs(shape, seed, dtype=torch.bfloat16):
    """N(0,1) with 1 % of the elements scaled by 8 (the FP8 workload's input recipe)."""
    g = torch.Generator().manual_seed(seed)
    outs = []
    for _ in range(3):
        x = torch.randn(shape, generator=g)
        x = torch.where(torch.rand(shape, generator=g) < 0.01, x * 8, x)
        outs.append(x.to(dtype))
    return outs


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("block", [128, 256, 512])
def test_block_quant_bit_exact(cuda, block, layout):
    from mindiesd.layers.quant import fa_block_quant_preprocess
    x = _outlier_inputs((1, 3, 1000, 128), seed=block)[0]
    x[0, 1, 256:384] = 0                      # an all-zero block
    xin = x if layout == "BNSD" else x.transpose(1, 2).contiguous()
    q, scale = fa_block_quant_preprocess(xin.to(cuda), block_size=block, layout=layout)
    codes, want_scale = oq.dynamic_block_quant(x, block, 128)
    assert q.dtype == torch.float8_e4m3fn and q.shape == (1, 3, 1000, 128)
    assert scale.shape == (1, 3, (1000 + block - 1) // block, 1) and scale.dtype == torch.float32
    assert torch.equal(scale.cpu(), want_scale)
    got = q.view(torch.uint8).cpu()
    same = got == codes
    # -0 / +0 codes are the same number
    zero = ((got & 0x7f) == 0) & ((codes & 0x7f) == 0)
    assert bool((same | zero).all()), f"{(~(same | zero)).sum().item()} codes differ"


def test_block_quant_fp16_and_errors(cuda):
    from mindiesd import ParametersInvalid
    from mindiesd.layers.quant import fa_block_quant_preprocess
    x = _outlier_inputs((2, 2, 300, 128), seed=3, dtype=torch.float16)[0]
    q, scale = fa_block_quant_preprocess(x.to(cuda))
    codes, want_scale = oq.dynamic_block_quant(x, 128, 128)
    assert torch.equal(scale.cpu()[..., 0], want_scale[..., 0])
    assert torch.equal(q.view(torch.uint8).cpu() & 0x7f, codes & 0x7f)
    with pytest.raises(ParametersInvalid):
        fa_block_quant_preprocess(x[0].to(cuda))
    with pytest.raises(ParametersInvalid):
        fa_block_quant_preprocess(x.to(cuda), block_size=64)


def test_v_per_channel_quant_bit_exact(cuda):
    from mindiesd.layers.quant.fp8_attention import quantize_v_per_channel
    v = _outlier_inputs((1, 2, 333, 128), seed=5)[2]
    v8t, vs = quantize_v_per_channel(v.to(cuda))
    codes, want = oq.per_channel_quant(v)
    assert torch.equal(vs.cpu(), want)
    assert v8t.shape == (1, 2, 128, 384)
    # undo the kernel's layout: position 32*h + j of each 64-key group holds key 32*(j/16) + 8*((j%16)/4) + 4*h + j%4
    pos = np.empty(64, dtype=np.int64)
    for h in range(2):
        for j in range(32):
            pos[32 * (j // 16) + 8 * ((j % 16) // 4) + 4 * h + j % 4] = 32 * h + j
    got = v8t.cpu().numpy().reshape(1, 2, 128, 6, 64)[..., pos].reshape(1, 2, 128, 384).transpose(0, 1, 3, 2)
    assert np.array_equal(got[:, :, :333] & 0x7f, codes.numpy() & 0x7f)
    assert (got[:, :, 333:] & 0x7f == 0).all(), "padding keys must be zero"


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("prescale", [1.0, 0.12751743])
def test_pow2_block_quant_bit_exact(cuda, prescale, layout):
    """Power-of-two block scales (+ a factor folded into x): the recipe of the log2-domain attention kernel."""
    from mindiesd.layers.quant.block_quant import _block_quant
    x = _outlier_inputs((1, 3, 1000, 128), seed=17)[0]
    x[0, 1, 256:384] = 0
    x[0, 2, :128] = 448.0 * 4                 # amax / 448 already a power of two: must not be doubled
    xin = x if layout == "BNSD" else x.transpose(1, 2).contiguous()
    q, scale = _block_quant(xin.to(cuda), 128, layout, prescale, True)
    codes, want_scale = oq.dynamic_block_quant(x, 128, 128, prescale, True)
    assert torch.equal(scale.cpu(), want_scale[..., 0])
    frac = np.frexp(scale.cpu().numpy())[0]
    assert (frac == 0.5).all(), "scales must be powers of two"
    got = q.cpu()
    zero = ((got & 0x7f) == 0) & ((codes & 0x7f) == 0)
    assert bool(((got == codes) | zero).all())
    if prescale == 1.0:
        assert scale[0, 2, 0].item() == 4.0


@pytest.mark.parametrize("p_rule", ["linear", "exp2"])
@pytest.mark.parametrize("recipe", ["pow2", "amax"])
@pytest.mark.parametrize("layout,s", [("BNSD", 1024), ("BNSD", 1100), ("BSND", 700)])
def test_fp8_attention_vs_oracle(cuda, layout, s, recipe, p_rule):
    from mindiesd.layers.quant import fp8_attention_forward
    q, k, v = _outlier_inputs((1, 3, s, 128), seed=s)
    want = oq.fp8_attention(q, k, v, pow2=recipe == "pow2")
    args = (q, k, v) if layout == "BNSD" else tuple(t.transpose(1, 2).contiguous() for t in (q, k, v))
    out = fp8_attention_forward(*(t.to(cuda) for t in args), layout=layout, recipe=recipe, p_rule=p_rule).cpu()
    out = out if layout == "BNSD" else out.transpose(1, 2)
    assert out.dtype == torch.bfloat16 and out.shape == q.shape
    cos = cosine(out, want)
    err = (out.float() - want.float()).abs()
    print(f"fp8 attention S={s} {layout} {recipe} {p_rule}: cosine {cos:.6f}, max-abs {err.max():.4f}, mean-abs {err.mean():.5f}, "
          f"output rms {want.float().pow(2).mean().sqrt():.4f}")
    assert cos >= 0.999, f"cosine {cos}"
    # coarse guard against gross outliers: E4M3 probabilities carry 2^-4 relative noise per element
    assert err.max() < 0.2 * want.float().abs().max()
    # against the oracle that re-quantises P the way the kernel does (same tiles, same reference rule, same
    # rounding): what is left is the summation order, the hardware's exp2 and a probability now and then landing on
    # the neighbouring E4M3 number
    mirror = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", requant_p=True, p_rule=p_rule)
    cos_m = cosine(out, mirror)
    err_m = (out.float() - mirror.float()).abs()
    print(f"   vs the P-requantising oracle: cosine {cos_m:.7f}, max-abs {err_m.max():.5f}")
    assert cos_m >= 0.99999, f"cosine {cos_m}"
    assert err_m.max() <= 2.0 ** -6 * max(1.0, want.float().abs().max().item())


@pytest.mark.parametrize("recipe", ["pow2", "amax"])
@pytest.mark.parametrize("sq,skv", [(700, 1100), (1300, 300), (130, 2049)])
def test_fp8_attention_unequal_query_and_key_lengths(cuda, sq, skv, recipe):
    """Cross attention: the query and key / value sequences have lengths of their own."""
    from mindiesd.layers.quant import fp8_attention_forward
    q, _, _ = _outlier_inputs((1, 2, sq, 128), seed=sq)
    _, k, v = _outlier_inputs((1, 2, skv, 128), seed=skv)
    want = oq.fp8_attention(q, k, v, pow2=recipe == "pow2")
    out = fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), layout="BNSD", recipe=recipe).cpu()
    assert out.shape == q.shape
    assert cosine(out, want) >= 0.999
    mirror = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", requant_p=True, p_rule="linear")
    assert cosine(out, mirror) >= 0.99999
    assert (out.float() - mirror.float()).abs().max() <= 2.0 ** -6 * max(1.0, want.float().abs().max().item())


@pytest.mark.parametrize("recipe", ["pow2", "amax"])
@pytest.mark.parametrize("s", [1100, 640])
def test_fp8_attention_k_scale_per_256_tokens(cuda, s, recipe):
    """K quantised per 256-token block (the K recipe of the reference's FP8RotateQuantFA, layer.py:297-302): scales from
    fa_block_quant_preprocess(block_size=256), the kernel takes one scale for two key tiles."""
    from mindiesd import ParametersInvalid
    from mindiesd.layers.quant import fp8_attention_forward
    q, k, v = _outlier_inputs((1, 2, s, 128), seed=s + 1)
    k[:, :, 256:512] *= 4.0                  # neighbouring 256-blocks with scales far apart
    out = fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), recipe=recipe, k_block=256).cpu()
    want = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", k_block=256)
    mirror = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", requant_p=True, k_block=256)
    assert cosine(out, want) >= 0.999 and cosine(out, mirror) >= 0.99999
    # a different quantisation from the per-128 one - except with power-of-two scales, where a coarser block only
    # shifts exponents and the dequantised values stay the same
    other = fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), recipe=recipe).cpu()
    assert torch.equal(out, other) == (recipe == "pow2")
    with pytest.raises(ParametersInvalid):
        fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), k_block=64)
    with pytest.raises(ParametersInvalid):
        fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), k_block=256,
                              k_rot=torch.eye(128, dtype=torch.bfloat16, device=cuda))


@pytest.mark.parametrize("p_rule", ["linear", "exp2"])
@pytest.mark.parametrize("recipe", ["pow2", "amax"])
def test_fp8_attention_scores_far_below_zero(cuda, recipe, p_rule):
    """q near +8, k near -8: every score lies hundreds of units below zero, the first key tile moves the running
    maximum far down."""
    from mindiesd.layers.quant import fp8_attention_forward
    g = torch.Generator().manual_seed(21)
    shape = (1, 2, 1100, 128)
    q = (8.0 + 0.5 * torch.randn(shape, generator=g)).to(torch.bfloat16)
    k = (-8.0 + 0.5 * torch.randn(shape, generator=g)).to(torch.bfloat16)
    v = torch.randn(shape, generator=g).to(torch.bfloat16)
    want = oq.fp8_attention(q, k, v, pow2=recipe == "pow2", requant_p=True, p_rule=p_rule)
    out = fp8_attention_forward(q.to(cuda), k.to(cuda), v.to(cuda), layout="BNSD", recipe=recipe, p_rule=p_rule).cpu()
    assert not torch.isnan(out.float()).any()
    assert cosine(out, want) >= 0.999


@pytest.mark.parametrize("layout,dtype", [("BNSD", torch.bfloat16), ("BSND", torch.bfloat16), ("BNSD", torch.float16)])
def test_rotation_fused_into_block_quant(cuda, layout, dtype):
    """x @ rot -> 16-bit -> block quantisation in one kernel vs matmul + quantisation on the CPU.  The two
    sides sum the 128 products of an element in different orders, so a rounded value may now and then land
    on the neighbouring 16-bit number: scales within one 16-bit ulp, at least 99.5 % of the codes identical,
    the rest one code step apart."""
    from mindiesd.layers.quant.block_quant import _rot_block_quant
    g = torch.Generator().manual_seed(21)
    rot, _ = torch.linalg.qr(torch.randn(128, 128, generator=g))
    rot = rot.to(dtype)
    x = _outlier_inputs((2, 3, 333, 128), seed=22)[0].to(dtype)
    want_c, want_s = oq.rot_block_quant(x, rot, 128)
    xin = x if layout == "BNSD" else x.transpose(1, 2).contiguous()
    codes, scale = _rot_block_quant(xin.to(cuda), rot.to(cuda), layout)
    codes, scale = codes.cpu(), scale.cpu()
    assert codes.shape == (2, 3, 333, 128) and scale.shape == (2, 3, 3)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert torch.allclose(scale, want_s.reshape(2, 3, 3), rtol=2 * ulp, atol=0)
    same = (codes == want_c)
    assert same.float().mean() >= 0.995, same.float().mean()
    diff = (torch.from_numpy(oq.e4m3_decode(codes.numpy())) - torch.from_numpy(oq.e4m3_decode(want_c.numpy()))).abs()
    step = torch.from_numpy(oq.e4m3_decode(want_c.numpy())).abs().clamp(min=2.0 ** -6) * 2.0 ** -3
    assert bool((diff <= 1.01 * step).all())
    # identity rotation: exactly the plain block quantisation
    from mindiesd.layers.quant.block_quant import _block_quant
    eye = torch.eye(128, dtype=dtype)
    c1, s1 = _rot_block_quant(xin.to(cuda), eye.to(cuda), layout)
    c0, s0 = _block_quant(xin.to(cuda), 128, layout)
    assert torch.equal(c1, c0) and torch.equal(s1, s0)


def test_fp8_rotate_quant_fa_module(cuda):
    """The reference's module shape (mindiesd/quantization/layer.py:274-324): orthogonal rotations
    leave q.k unchanged, so the output must stay close to unquantised attention."""
    from mindiesd.quantization import FP8RotateQuantFA
    from oracle.attention import attention_math
    g = torch.Generator().manual_seed(9)
    rot_q, _ = torch.linalg.qr(torch.randn(128, 128, generator=g))
    weights = {"blk.attn.q_rot": rot_q.to(torch.bfloat16).to(cuda), "blk.attn.k_rot": rot_q.to(torch.bfloat16).to(cuda)}
    mod = FP8RotateQuantFA(prefix="blk.attn", weights=weights)
    q, k, v = _outlier_inputs((1, 600, 2, 128), seed=11)
    out = mod(q.to(cuda), k.to(cuda), v.to(cuda), layout="BSND").cpu()
    ref = attention_math(q, k, v, None, 128 ** -0.5, head_first=False)
    assert out.shape == q.shape and cosine(out, ref) > 0.995
    with pytest.raises(ValueError):
        mod(q.to(cuda), k.to(cuda), v.to(cuda), layout="SBH")


def test_ops_match_the_python_functions_and_trace(cuda):
    """torch.ops.mindiesd.{fa_block_quant, fp8_attention_fwd, mxfp8_gemm_swiglu, rf_block_mask} give what the Python
    entry points give, and a function built from them compiles as one graph (fake implementations present)."""
    import mindiesd  # noqa: F401
    from mindiesd.layers.flash_attn import rainfusion as rf
    from mindiesd.layers.quant import fa_block_quant_preprocess, fp8_attention_forward, mx_quantize, mxfp8_matmul
    q, k, v = (t.to(cuda) for t in _outlier_inputs((1, 2, 700, 128), seed=11))
    codes, scale = torch.ops.mindiesd.fa_block_quant(q, 128, "BNSD")
    c2, s2 = fa_block_quant_preprocess(q, block_size=128)
    assert torch.equal(codes.view(torch.uint8), c2.view(torch.uint8)) and torch.equal(scale, s2)
    out = torch.ops.mindiesd.fp8_attention_fwd(q, k, v, 128 ** -0.5)
    assert torch.equal(out, fp8_attention_forward(q, k, v))
    x = torch.randn(5, 30, 256, device=cuda).to(torch.bfloat16)
    wq, ws = mx_quantize((torch.randn(512, 256, device=cuda) * 0.05).to(torch.bfloat16))
    y = torch.ops.mindiesd.mxfp8_gemm_swiglu(x, wq, ws)
    xq, xs = mx_quantize(x.reshape(-1, 256))
    assert torch.equal(y, mxfp8_matmul(xq, xs, wq, ws, None, torch.bfloat16, True).view(5, 30, 256))
    grid = (2, 24, 24)
    qq, kk, vv = (torch.randn(1, 2, 2 * 24 * 24, 128, device=cuda).to(torch.bfloat16) for _ in range(3))
    _, _, _, pool = rf.do_tensor_rearrange_pooling(qq, kk, vv, 0, 128, grid, grid, "BNSD")
    m = torch.ops.mindiesd.rf_block_mask(pool, 0, 0.6, 128 ** -0.5, list(grid))
    assert torch.equal(m, rf.get_blockwise_mask(pool, 0, 0.6, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True))

    def fn(a, b, c, xx):
        return torch.ops.mindiesd.fp8_attention_fwd(a, b, c, 128 ** -0.5), torch.ops.mindiesd.mxfp8_gemm_swiglu(xx, wq, ws)

    o1, o2 = torch.compile(fn, backend="eager", fullgraph=True)(q, k, v, x)
    assert torch.equal(o1, out) and torch.equal(o2, y)
