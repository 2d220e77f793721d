"""``attention_forward``: the dense attention front door (mindiesd/layers/flash_attn/attention_forward.py:24-128)."""
import os

import torch

from .attention_func import (attention_math, get_attention_function, get_attention_function_runtime,
                             get_attention_function_static)
from .common import AttentionParam
from ...utils.exception import ParametersInvalid

SUPPORTED_FA_TYPES = ("hip_flash_attn", "prompt_flash_attn", "fused_attn_score", "ascend_laser_attention")


def attention_forward(query, key, value, attn_mask=None, scale=None, fused=True, head_first=False, **kwargs):
    """Attention forward.  ``head_first=False``: q/k/v are [B, S, N, D]; ``True``: [B, N, S, D].
    The output has the layout and dtype of ``query``.

    Args:
        attn_mask: [Sq|1, Skv] or [B|1, N|1, Sq|1, Skv] (query dimension 1: one row for all queries), True / non-zero = attend.
        scale: float softmax scale, default head_dim ** -0.5.
        fused: True runs the HIP flash-attention kernel, False the unfused torch math.
        kwargs: ``opt_mode`` in {'runtime' (default), 'static', 'manual'}; with 'manual',
            ``op_type`` (any of the reference's names or 'hip_flash_attn'; env ``MINDIE_SD_FA_TYPE``
            overrides it) and ``layout`` in {'BNSD', 'BSND', 'BSH'}.
    """
    check_input_params((query, key, value, attn_mask, scale, fused))
    if head_first:
        attn_param = AttentionParam(query.shape[0], query.shape[1], query.shape[-1], query.shape[2], key.shape[2],
                                    query.dtype, head_first)
    else:
        attn_param = AttentionParam(query.shape[0], query.shape[-2], query.shape[-1], query.shape[1], key.shape[1],
                                    query.dtype, head_first)
    if scale is None:
        scale = attn_param.head_dim ** -0.5
    if not fused:
        return attention_math(query, key, value, attn_mask, scale, head_first)

    opt_mode = kwargs.get("opt_mode", "runtime")
    if opt_mode == "static":
        attn_func = get_attention_function_static(attn_param)
    elif opt_mode == "manual":
        op_type = os.getenv("MINDIE_SD_FA_TYPE") or kwargs.get("op_type", "fused_attn_score")
        if op_type not in SUPPORTED_FA_TYPES:
            raise ParametersInvalid(f"Unsupported FA type: '{op_type}'. Supported values: {set(SUPPORTED_FA_TYPES)}")
        attn_func = get_attention_function(attn_param, op_type, kwargs.get("layout", "BNSD"))
    elif opt_mode == "runtime":
        attn_func = get_attention_function_runtime(attn_param, query, key, value, attn_mask, scale)
    else:
        raise ParametersInvalid(f"The input 'opt_mode':{opt_mode} is invalid. "
                                f"The list of supported options is ['runtime', 'static', 'manual']")
    return attn_func(query, key, value, attn_mask, scale)


def check_input_params(input_params):
    """Type / rank checks of attention_forward.py:92-111."""
    query, key, value, attn_mask, scale, fused = input_params
    for name, t in (("query", query), ("key", key), ("value", value)):
        if not isinstance(t, torch.Tensor):
            raise ParametersInvalid(f"The data type of input {name} must be torch.Tensor, but got {type(t)}.")
    for name, t in (("query", query), ("key", key), ("value", value)):
        if t.dim() != 4:
            raise ParametersInvalid(f"The dimensional of input {name} must be 4, but got {t.dim()}.")
    if not isinstance(fused, bool):
        raise ParametersInvalid(f"The data type of input fused must be bool, but got {type(fused)}.")
    if attn_mask is not None and not isinstance(attn_mask, torch.Tensor):
        raise ParametersInvalid(f"The data type of input attn_mask must be torch.Tensor, but got {type(attn_mask)}.")
    if scale is not None and not isinstance(scale, float):
        raise ParametersInvalid(f"The data type of input scale must be float, but got {type(scale)}.")
