"""Unfused attention math and kernel selection (mindiesd/layers/flash_attn/attention_func.py).

``attention_math`` is the reference's ``fused=False`` path: plain torch ops on whatever device the
tensors live on.  It is part of the public API and is only ever taken when the caller asks for it;
fused calls never fall back to it.
"""
from functools import partial

import torch

from .attention_operate import device_mi355x_op
from .common import AttentionParam, lru_cache_by_attn_param
from . import hip_flash_attn  # noqa: F401  (registers the kernel)
from ...utils.exception import ParametersInvalid
from ...utils.logs import logger

DEFAULT_OP = "hip_flash_attn"
ATTN_DICT = {}  # static table: AttentionParam hash -> (op_type, layout); empty = default everywhere


def attention_math(query, key, value, attn_mask, scale, head_first=False):
    """attention_func.py:32-55, including its rounding points (q*scale, QK^T and P in the input dtype)."""
    if not head_first:
        query, key, value = query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2)
    dtype = query.dtype
    q_seqlen, kv_seqlen = query.size(-2), key.size(-2)
    attn = ((query * scale) @ key.transpose(-2, -1)).to(torch.float32)
    if attn_mask is not None:
        if attn_mask.dim() not in (2, 4) or attn_mask.size(-2) != q_seqlen or attn_mask.size(-1) != kv_seqlen:
            raise ParametersInvalid("The attn_mask must be a 2D tensor with shape [q_seqlen, kv_seqlen],"
                                    " or a 4D tensor with shape [batch_size, num_heads, q_seqlen, kv_seqlen]")
        bias = torch.zeros(attn_mask.shape, dtype=dtype, device=query.device)
        bias.masked_fill_(attn_mask.logical_not(), float("-inf"))
        attn = attn + bias
    out = torch.softmax(attn, dim=-1).to(dtype) @ value
    return out if head_first else out.transpose(1, 2)


def get_attention_function(attn_param: AttentionParam, op_type, layout):
    """Bind ``attn_param`` to the requested kernel/layout after validating both (attention_func.py:73-100)."""
    registry = device_mi355x_op.get_all()
    if op_type not in registry:
        raise ParametersInvalid(f"The 'op_type':{op_type} is not supported. "
                                f"The list of supported options is {list(registry.keys())}")
    op = registry[op_type]
    if layout not in op.supported_layout:
        raise ParametersInvalid(f"The 'layout':{layout} is not supported. "
                                f"The list of supported options is {op.supported_layout}")
    if attn_param.dtype not in op.supported_dtype:
        raise ParametersInvalid(f"The input dtype:{attn_param.dtype} is not supported. "
                                f"The list of supported options is {op.supported_dtype}")
    if not op.is_supported_shape(attn_param):
        raise ParametersInvalid(f"The input shape is not supported by '{op_type}': {attn_param.to_str()}")
    return partial(getattr(op, op.layout_to_func[layout]), attn_param)


def get_attention_function_static(attn_param: AttentionParam):
    op_type, layout = ATTN_DICT.get(attn_param.to_hash(), (DEFAULT_OP, "BNSD"))
    return get_attention_function(attn_param, op_type, layout)


@lru_cache_by_attn_param(maxsize=512)
def get_attention_function_runtime(attn_param: AttentionParam, query=None, key=None, value=None, attn_mask=None,
                                   scale=None):
    """The reference times every registered kernel x layout on the first call of a shape
    (attention_func.py:103-171).  One stride-generic kernel is registered here, so the choice needs
    no timing run; the per-shape LRU cache is kept."""
    logger.debug("select attention kernel for %s", attn_param.to_str())
    layout = "BNSD" if attn_param.head_first else "BSND"
    return get_attention_function(attn_param, DEFAULT_OP, layout)
