"""FP8 block quantisation of attention operands (mindiesd/layers/quant/block_quant.py:19-48)."""
import torch

from ... import _native
from ...utils.exception import ParametersInvalid
from ..flash_attn.hip_flash_attn import HEAD_DIM, _strides_bns


def _block_quant(x, block_size, layout, prescale=1.0, pow2=False):
    """x 4-D bf16/fp16 GPU tensor in ``layout`` -> (uint8 E4M3 codes [B,N,S,D] contiguous, fp32 scale
    [B,N,ceil(S/block_size)]).  ``prescale`` multiplies x first; ``pow2`` rounds each scale up to a power of two
    (x * prescale ~ codes * scale either way)."""
    if x.dtype not in _native.DTYPE_CODE or not x.is_cuda:
        raise ParametersInvalid(f"fa block quant needs a bf16/fp16 GPU tensor, but got {x.dtype} on {x.device}.")
    if x.shape[-1] != HEAD_DIM:
        raise ParametersInvalid(f"fa block quant supports head_dim == {HEAD_DIM}, but got {x.shape[-1]}.")
    if block_size not in (128, 256, 512):
        raise ParametersInvalid(f"block_size supports 128/256/512, but got {block_size}.")
    ok = x.stride(-1) == 1 and x.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in x.stride()[:-1])
    x = x if ok else x.contiguous()
    b, n, s = (x.shape[0], x.shape[1], x.shape[2]) if layout == "BNSD" else (x.shape[0], x.shape[2], x.shape[1])
    q = torch.empty((b, n, s, HEAD_DIM), dtype=torch.uint8, device=x.device)
    scale = torch.empty((b, n, (s + block_size - 1) // block_size), dtype=torch.float32, device=x.device)
    with _native.on_device(x.device):
        rc = _native.lib().mindiesd_fa_block_quant(x.data_ptr(), q.data_ptr(), scale.data_ptr(),
                                                   _native.DTYPE_CODE[x.dtype], b, n, s, HEAD_DIM,
                                                   *_strides_bns(x, layout), block_size, float(prescale),
                                                   int(bool(pow2)), _native.stream_ptr(x.device))
    _native.check(rc, "mindiesd_fa_block_quant")
    return q, scale


def _rot_block_quant(x, rot, layout, prescale=1.0, pow2=False):
    """(x @ rot) rounded to x.dtype, then quantised per (head, 128 tokens) in one pass over x.
    x 4-D bf16/fp16 GPU tensor in ``layout``, rot [128, 128]; returns (uint8 codes [B,N,S,D], fp32 scale
    [B,N,ceil(S/128)])."""
    if x.dtype not in _native.DTYPE_CODE or not x.is_cuda:
        raise ParametersInvalid(f"fa block quant needs a bf16/fp16 GPU tensor, but got {x.dtype} on {x.device}.")
    if x.shape[-1] != HEAD_DIM or tuple(rot.shape) != (HEAD_DIM, HEAD_DIM):
        raise ParametersInvalid(f"rotation + block quant supports head_dim == {HEAD_DIM} and a [{HEAD_DIM}, {HEAD_DIM}] "
                                f"rotation, but got {x.shape[-1]} and {tuple(rot.shape)}.")
    ok = x.stride(-1) == 1 and x.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in x.stride()[:-1])
    x = x if ok else x.contiguous()
    rot_t = rot.to(device=x.device, dtype=x.dtype).t().contiguous()
    b, n, s = (x.shape[0], x.shape[1], x.shape[2]) if layout == "BNSD" else (x.shape[0], x.shape[2], x.shape[1])
    q = torch.empty((b, n, s, HEAD_DIM), dtype=torch.uint8, device=x.device)
    scale = torch.empty((b, n, (s + 127) // 128), dtype=torch.float32, device=x.device)
    with _native.on_device(x.device):
        rc = _native.lib().mindiesd_fa_rot_block_quant(x.data_ptr(), rot_t.data_ptr(), q.data_ptr(), scale.data_ptr(),
                                                       _native.DTYPE_CODE[x.dtype], b, n, s, HEAD_DIM,
                                                       *_strides_bns(x, layout), float(prescale), int(bool(pow2)),
                                                       _native.stream_ptr(x.device))
    _native.check(rc, "mindiesd_fa_rot_block_quant")
    return q, scale


def fa_block_quant_preprocess(input_tensor, block_size=128, dst_type=torch.float8_e4m3fn, **kwargs):
    """Quantise q, k or v for FP8 attention.  ``layout`` kwarg: 'BNSD' (default) or 'BSND'.

    Returns ``(x_q, scale)``: ``x_q`` float8_e4m3fn [B, N, S, D] (always head-first, as in the
    reference, which transposes BSND inputs before quantising) and ``scale`` fp32
    [B, N, ceil(S / block_size), 1] with ``x ~ x_q * scale`` per (head, block_size tokens, all 128
    channels).  The reference squeezes the batch dimension for its vendor op, i.e. assumes B == 1;
    any B works here."""
    if not isinstance(input_tensor, torch.Tensor) or input_tensor.dim() != 4:
        raise ParametersInvalid(f"fa block quant preprocess only support qkv quant, dim = 4, "
                                f"but got {getattr(input_tensor, 'dim', lambda: None)()}.")
    if dst_type != torch.float8_e4m3fn:
        raise ParametersInvalid(f"dst_type only supports torch.float8_e4m3fn, but got {dst_type}.")
    layout = kwargs.get("layout", "BNSD")
    if layout not in ("BNSD", "BSND"):
        raise ParametersInvalid(f"layout must be 'BNSD' or 'BSND', but got {layout}.")
    q, scale = _block_quant(input_tensor, block_size, layout)
    return q.view(torch.float8_e4m3fn), scale.unsqueeze(-1)
