"""MXFP8 (OCP MX: E4M3 + one E8M0 scale per 32 elements along K) quantisation and GEMM, with an
optional fused SwiGLU epilogue, on the MI355X scaled fp8 matrix cores.

Counterparts of ``torch_npu.npu_dynamic_mx_quant`` and ``torch_npu.npu_quant_matmul(...,
group_sizes=[1, 1, 32])`` as used by the reference's MXFP8 linear layer
(mindiesd/quantization/layer.py:334-361)."""
import torch

from ... import _native
from ...utils.exception import ParametersInvalid


def mx_quantize(x):
    """[M, K] bf16/fp16 (row stride a multiple of 8, K % 32 == 0) ->
    (float8_e4m3fn [M, K], float8_e8m0fnu [M, K/32])."""
    if not isinstance(x, torch.Tensor) or x.dim() != 2 or not x.is_cuda or x.dtype not in _native.DTYPE_CODE:
        raise ParametersInvalid("mx_quantize needs a 2-D bf16/fp16 GPU tensor.")
    m, k = x.shape
    if k % 32 != 0:
        raise ParametersInvalid(f"mx_quantize needs K % 32 == 0, but got K = {k}.")
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    q = torch.empty((m, k), dtype=torch.uint8, device=x.device)
    e = torch.empty((m, k // 32), dtype=torch.uint8, device=x.device)
    with _native.on_device(x.device):
        rc = _native.lib().mindiesd_mx_quant(x.data_ptr(), q.data_ptr(), e.data_ptr(), _native.DTYPE_CODE[x.dtype], m, k,
                                             x.stride(0), _native.stream_ptr(x.device))
    _native.check(rc, "mindiesd_mx_quant")
    return q.view(torch.float8_e4m3fn), e.view(torch.float8_e8m0fnu)


def _as_u8(t, what, shape):
    if t.dtype not in (torch.uint8, torch.float8_e4m3fn, torch.float8_e8m0fnu) or not t.is_cuda:
        raise ParametersInvalid(f"{what} must be a 1-byte (fp8 / e8m0 / uint8) GPU tensor, but got {t.dtype}.")
    t = t.reshape(shape)
    return t.contiguous().view(torch.uint8)


def mxfp8_matmul(x_q, x_scale, w_q, w_scale, bias=None, out_dtype=torch.bfloat16, swiglu=False):
    """``act(x @ w.T + bias)`` on MX-quantised operands: x_q [M, K] E4M3, x_scale [M, K/32] E8M0,
    w_q [Nw, K], w_scale [Nw, K/32] (also accepted as [Nw, K/64, 2], the reference's storage shape).
    ``swiglu=True``: w = [gate rows | up rows], result [M, Nw/2] = silu(gate) * up; else [M, Nw]."""
    if x_q.dim() != 2 or w_q.dim() != 2 or x_q.shape[1] != w_q.shape[1]:
        raise ParametersInvalid("mxfp8_matmul needs x_q [M, K] and w_q [N, K].")
    m, k = x_q.shape
    nw = w_q.shape[0]
    if k % 128 != 0:
        raise ParametersInvalid(f"mxfp8_matmul needs K % 128 == 0, but got K = {k}.")
    if nw % (16 if swiglu else 8) != 0:
        raise ParametersInvalid(f"mxfp8_matmul needs the weight row count to be a multiple of "
                                f"{16 if swiglu else 8}, but got {nw}.")
    if out_dtype not in _native.DTYPE_CODE:
        raise ParametersInvalid(f"out_dtype must be bf16 or fp16, but got {out_dtype}.")
    xq, wq = _as_u8(x_q, "x_q", (m, k)), _as_u8(w_q, "w_q", (nw, k))
    xs, ws = _as_u8(x_scale, "x_scale", (m, k // 32)), _as_u8(w_scale, "w_scale", (nw, k // 32))
    if bias is not None:
        bias = bias.to(device=xq.device, dtype=torch.float32).contiguous()
        if bias.numel() != nw:
            raise ParametersInvalid("bias must have one entry per weight row.")
    out = torch.empty((m, nw // 2 if swiglu else nw), dtype=out_dtype, device=xq.device)
    with _native.on_device(xq.device):
        rc = _native.lib().mindiesd_mxfp8_gemm(xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(),
                                               bias.data_ptr() if bias is not None else None, out.data_ptr(),
                                               _native.DTYPE_CODE[out_dtype], m, k, nw, int(bool(swiglu)),
                                               _native.stream_ptr(xq.device))
    _native.check(rc, "mindiesd_mxfp8_gemm")
    return out


def mxfp8_gemm_swiglu(x, w_q, w_scale, bias=None, out_dtype=None):
    """DiT FFN up-projection: quantise the activations ``x`` [..., K] on the fly, multiply with the
    MX-quantised weight [gate | up] ([2F, K]) and return ``silu(gate) * up`` [..., F]."""
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    xq, xs = mx_quantize(x2)
    out = mxfp8_matmul(xq, xs, w_q, w_scale, bias, out_dtype or x.dtype, swiglu=True)
    return out.view(*lead, out.shape[-1])
