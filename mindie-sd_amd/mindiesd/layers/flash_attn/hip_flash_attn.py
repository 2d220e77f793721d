"""The MI355X attention kernel behind ``attention_forward``.

Takes the place of the reference's vendor-op wrappers (prompt_flash_attn.py:22-130,
fused_attn_score.py:22-131, ascend_laser_attention.py:38-119).  Those normalise the layout with
transposes / reshapes before calling a layout-specific NPU kernel; the HIP kernel takes explicit
batch / head / token strides, so BNSD, BSND and BSH inputs all run in place without a copy.
"""
import torch

from .attention_operate import AttentionOperateBase, register_op_mi355x
from .common import AttentionParam
from ... import _native
from ...utils.exception import ParametersInvalid

HEAD_DIM = 128


def _strides_bns(t, layout):
    """(batch, head, token) element strides of a 4-D tensor in ``layout`` with a contiguous last dim."""
    if t.stride(-1) != 1:
        raise ParametersInvalid("The last dimension of query/key/value must be contiguous.")
    if layout == "BNSD":
        return t.stride(0), t.stride(1), t.stride(2)
    return t.stride(0), t.stride(2), t.stride(1)


def flash_attention(query, key, value, scale, layout="BNSD", return_lse=False):
    """softmax(scale * Q K^T) V on the GPU.  ``layout`` is 'BNSD' or 'BSND'; the output has the
    input's layout and dtype.  Grouped-query attention is supported (N % N_kv == 0)."""
    for name, t in (("query", query), ("key", key), ("value", value)):
        if not t.is_cuda:
            raise ParametersInvalid(f"The fused attention kernel needs GPU tensors, but {name} is on {t.device}.")
    if query.dtype not in _native.DTYPE_CODE or key.dtype != query.dtype or value.dtype != query.dtype:
        raise ParametersInvalid(f"The fused attention kernel supports bf16/fp16 with equal q/k/v dtypes, "
                                f"but got {query.dtype}, {key.dtype}, {value.dtype}.")
    if layout == "BNSD":
        b, n, sq, d = query.shape
        nkv, skv = key.shape[1], key.shape[2]
    else:
        b, sq, n, d = query.shape
        skv, nkv = key.shape[1], key.shape[2]
    if d != HEAD_DIM or key.shape[-1] != d or value.shape[-1] != d:
        raise ParametersInvalid(f"The fused attention kernel supports head_dim == {HEAD_DIM}, but got {d}.")
    if key.shape != value.shape or key.shape[0] != b or n % nkv != 0:
        raise ParametersInvalid("Inconsistent query/key/value shapes.")
    fix = lambda t: t if (t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1])
                          and t.data_ptr() % 16 == 0) else t.contiguous()
    query, key, value = fix(query), fix(key), fix(value)
    out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    lse = torch.empty((b, n, sq), dtype=torch.float32, device=query.device) if return_lse else None
    with torch.cuda.device(query.device):
        rc = _native.lib().mindiesd_flash_attention_fwd(
            query.data_ptr(), key.data_ptr(), value.data_ptr(), out.data_ptr(),
            lse.data_ptr() if lse is not None else None, _native.DTYPE_CODE[query.dtype],
            b, n, nkv, sq, skv, d,
            *_strides_bns(query, layout), *_strides_bns(key, layout), *_strides_bns(value, layout),
            *_strides_bns(out, layout), float(scale), _native.stream_ptr(query.device))
    _native.check(rc, "mindiesd_flash_attention_fwd")
    return (out, lse) if return_lse else out


@register_op_mi355x("hip_flash_attn", "prompt_flash_attn", "fused_attn_score", "ascend_laser_attention")
class HipFlashAttention(AttentionOperateBase):
    """Registered under its own name and under the reference's three op names, so call sites that
    pass ``op_type='fused_attn_score'`` etc. (attention_forward.py:72-80) keep working."""
    supported_layout = ["BNSD", "BSND", "BSH"]
    supported_dtype = [torch.bfloat16, torch.float16]

    @classmethod
    def is_supported_shape(cls, attn_param: AttentionParam) -> bool:
        return attn_param.head_dim == HEAD_DIM

    @classmethod
    def _run(cls, attn_param, query, key, value, mask, scale):
        if mask is not None:
            raise ParametersInvalid("attn_mask is not supported by the fused HIP kernel; "
                                    "call attention_forward(..., fused=False) for masked attention.")
        if scale is None:
            scale = attn_param.head_dim ** -0.5
        return flash_attention(query, key, value, scale, "BNSD" if attn_param.head_first else "BSND")

    # The kernel is stride-generic, so the three "layouts" of the reference differ only in how the
    # caller's tensors are viewed: nothing is transposed or copied for any of them.
    @classmethod
    def forward_attn_bnsd(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)

    @classmethod
    def forward_attn_bsnd(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)

    @classmethod
    def forward_attn_bsh(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)
