"""GPU parity of the MXFP8 path vs the CPU oracle: MX quantisation bit-exact against the OCP MX
definition; GEMM (+ bias) and GEMM + SwiGLU against the dequantise -> exact GEMM oracle.  Stated
tolerance: cosine >= 0.999; since both sides multiply the same quantised numbers the match is in
fact limited only by fp32 accumulation and the 16-bit output rounding, which is asserted too."""
import pytest
import torch

from oracle import quant as oq
from oracle.attention import cosine

pytestmark = pytest.mark.gpu


def _rand(shape, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mx_quant_bit_exact(cuda, dtype):
    from mindiesd.layers.quant import mx_quantize
    x = _rand((300, 512), 1, dtype=dtype) * torch.logspace(-2, 2, 300)[:, None].to(dtype)
    x[7, 64:96] = 0
    q, e = mx_quantize(x.to(cuda))
    codes, e8 = oq.mx_quant(x)
    assert q.dtype == torch.float8_e4m3fn and e.dtype == torch.float8_e8m0fnu and e.shape == (300, 16)
    assert torch.equal(e.view(torch.uint8).cpu(), e8)
    assert torch.equal(q.view(torch.uint8).cpu() & 0x7f, codes & 0x7f)
    assert torch.equal((q.view(torch.uint8).cpu() >> 7)[codes & 0x7f != 0], (codes >> 7)[codes & 0x7f != 0])


@pytest.mark.parametrize("m,k,f", [(256, 512, 128), (300, 1024, 136), (1000, 256, 520)])
def test_gemm_swiglu_vs_oracle(cuda, m, k, f):
    from mindiesd.layers.quant import mx_quantize, mxfp8_gemm_swiglu
    x = _rand((m, k), 2)
    w = _rand((2 * f, k), 3, scale=0.05)
    wq, ws = mx_quantize(w.to(cuda))
    out = mxfp8_gemm_swiglu(x.to(cuda), wq, ws).cpu()
    want = oq.mxfp8_gemm_swiglu(x, w, torch.float32)
    assert out.shape == (m, f) and out.dtype == torch.bfloat16
    assert cosine(out, want) >= 0.999
    err = (out.float() - want).abs()
    assert (err <= 2.0 ** -7 * want.abs() + 1e-3).all(), f"max err {err.max()}"


def test_plain_gemm_with_bias_and_linear_module(cuda):
    from mindiesd.layers.quant import mx_quantize, mxfp8_matmul
    from mindiesd.quantization import W8A8MXFP8QuantLinear
    m, k, n = 520, 384, 264
    x = _rand((2, m // 2, k), 4)
    w = _rand((n, k), 5, scale=0.05)
    bias = _rand((n,), 6, dtype=torch.float32)
    wq, ws = mx_quantize(w.to(cuda))
    want = oq.mxfp8_gemm(x.reshape(m, k), w, bias).float()
    xq, xs = mx_quantize(x.reshape(m, k).to(cuda))
    out = mxfp8_matmul(xq, xs, wq, ws, bias.to(cuda), torch.bfloat16).cpu()
    assert out.shape == (m, n)
    assert ((out.float() - want).abs() <= 2.0 ** -7 * want.abs() + 1e-3).all()
    # reference-shaped module: weight_scale stored as [N, K/64, 2]
    weights = {"ffn.up.weight": wq, "ffn.up.weight_scale": ws.view(torch.uint8).reshape(n, k // 64, 2),
               "ffn.up.bias": bias.to(cuda)}
    lin = W8A8MXFP8QuantLinear(k, n, bias=True, weights=weights, prefix="ffn.up")
    y = lin(x.to(cuda))
    assert y.shape == (2, m // 2, n) and torch.equal(y.reshape(m, n).cpu(), out)


def test_gemm_errors(cuda):
    from mindiesd import ParametersInvalid
    from mindiesd.layers.quant import mx_quantize, mxfp8_matmul
    x = _rand((64, 96), 7)
    xq, xs = mx_quantize(x.to(cuda))
    with pytest.raises(ParametersInvalid):
        mxfp8_matmul(xq, xs, xq, xs)            # K not a multiple of 128
    with pytest.raises(ParametersInvalid):
        mx_quantize(_rand((4, 40), 8).to(cuda))  # K not a multiple of 32


def test_quantize_injected_layers_match_direct_calls(cuda, tmp_path):
    """quantize() on a toy block (descriptor + safetensors written here): the swapped-in linear equals the direct
    MXFP8 GEMM on the same tensors, the attached fa_quant equals the direct FP8 attention call."""
    import json
    import os
    from safetensors.torch import save_file
    from torch import nn
    from mindiesd import quantize
    from mindiesd.layers.quant import fp8_attention_forward, mx_quantize, mxfp8_matmul

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.up = nn.Linear(256, 512)
            self.attn = nn.Identity()

    g = torch.Generator().manual_seed(0)
    w = (torch.randn(512, 256, generator=g) * 0.05).to(torch.bfloat16).to(cuda)
    wq, ws = mx_quantize(w)
    bias = torch.randn(512, generator=g)
    rot = torch.linalg.qr(torch.randn(128, 128, generator=g))[0].to(torch.bfloat16).contiguous()
    weights = {"up.weight": wq.cpu(), "up.weight_scale": ws.view(torch.uint8).cpu().reshape(512, -1, 2).contiguous(),
               "up.bias": bias, "attn.q_rot": rot, "attn.k_rot": rot.clone()}
    des = {"model_quant_type": "W8A8_MXFP8", "up.weight": "W8A8_MXFP8", "attn.fa_q.scale": "FP8_DYNAMIC"}
    with open(os.path.join(tmp_path, "d.json"), "w") as f:
        json.dump(des, f)
    save_file(weights, os.path.join(tmp_path, "quant_model_weight_w8a8_mxfp8.safetensors"))
    model = quantize(Block(), os.path.join(str(tmp_path), "d.json")).to(cuda)
    x = torch.randn(3, 40, 256, generator=g).to(torch.bfloat16).to(cuda)
    got = model.up(x)
    xq, xs = mx_quantize(x.reshape(-1, 256))
    want = mxfp8_matmul(xq, xs, wq, ws, bias.to(cuda), torch.bfloat16, False).view(3, 40, 512)
    assert got.shape == (3, 40, 512) and torch.equal(got, want)
    q, k, v = (torch.randn(1, 2, 300, 128, generator=g).to(torch.bfloat16).to(cuda) for _ in range(3))
    a = model.attn.fa_quant(q, k, v, layout="BNSD")
    b = fp8_attention_forward(q, k, v, layout="BNSD", q_rot=rot.to(cuda), k_rot=rot.to(cuda))
    assert torch.equal(a, b)
