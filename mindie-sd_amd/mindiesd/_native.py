"""ctypes binding of ``plugin/libmindiesd_hip.so`` (C ABI declared in include/mindiesd_hip.h).

The library location mirrors the reference's ``<package>/plugin/libPTAExtensionOPS.so``
(mindiesd/layers/register_ops.py:24-44).  Importing the package never loads it; the first
fused call does, and a missing library is a hard error -- there is no CPU fallback.
"""
import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plugin", "libmindiesd_hip.so")
_lib = None

ERRORS = {
    1: "bad argument (null/misaligned pointer, non-positive size, unsupported dtype)",
    2: "unsupported shape or option",
    3: "workspace too small",
    4: "HIP launch failure",
}

c_int, c_ll, c_f, c_p, c_sz = ctypes.c_int, ctypes.c_longlong, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol of include/mindiesd_hip.h
SIGNATURES = {
    "mindiesd_flash_attention_fwd": (c_int, [c_p] * 5 + [c_int] * 7 + [c_ll] * 12 + [c_f, c_p]),
    "mindiesd_flash_attention_general_fwd": (c_int, [c_p] * 5 + [c_int] * 7 + [c_ll] * 12 + [c_f, c_p, c_int, c_p] + [c_ll] * 3 + [c_p]),
    "mindiesd_flash_attention_packed_fwd": (c_int, [c_p] * 4 + [c_int] * 7 + [c_ll] * 8 + [c_f, c_p, c_int, c_p]),
    "mindiesd_varlen_meta": (c_int, [c_p] * 2 + [c_int] * 5 + [c_p] * 2),
    "mindiesd_ada_block_sparse_attention_fwd": (c_int, [c_p] * 4 + [c_int] * 6 + [c_ll] * 12 + [c_f, c_p, c_p, c_int, c_int, c_p]),
    "mindiesd_sbe_scores_workspace_size": (c_sz, [c_int, c_int]),
    "mindiesd_sbe_scores": (c_int, [c_p, c_p, c_p] + [c_int] * 6 + [c_ll] * 6 + [c_f, c_int, c_p, c_sz, c_p]),
    "mindiesd_sbe_select": (c_int, [c_p, c_p, c_p] + [c_int] * 3 + [c_f, c_f, c_int, c_int, c_int, c_p]),
    "mindiesd_block_sparse_attention_fwd": (c_int, [c_p] * 5 + [c_int] * 7 + [c_ll] * 12 + [c_f, c_p, c_p, c_int, c_p, c_p]),
    "mindiesd_rf_rearrange_pool": (c_int, [c_p] * 7 + [c_int] * 5 + [c_ll] * 10 + [c_int] * 6 + [c_p]),
    "mindiesd_rf_block_mask": (c_int, [c_p, c_p] + [c_int] * 5 + [c_ll] * 3 + [c_f] + [c_int] * 4 + [c_p] * 3 + [c_int, c_p, c_p, c_p]),
    "mindiesd_mask_to_index": (c_int, [c_p, c_int, c_int, c_int, c_p, c_p, c_int, c_p]),
    "mindiesd_block_sparse_attention_gather_fwd": (c_int, [c_p] * 5 + [c_int] * 6 + [c_ll] * 12 + [c_f, c_p, c_p, c_int, c_p,
                                                                                            c_p]),
    "mindiesd_block_sparse_attention_paired_workspace_size": (c_sz, [c_int] * 4),
    "mindiesd_block_sparse_attention_paired_fwd": (c_int, [c_p] * 5 + [c_int] * 7 + [c_ll] * 12 + [c_f, c_p, c_p, c_p, c_sz,
                                                                                          c_p]),
    "mindiesd_block_sparse_attention_general_fwd": (c_int, [c_p] * 5 + [c_int] * 7 + [c_ll] * 12 + [c_f, c_p, c_p, c_int, c_p,
                                                                                           c_int, c_int, c_p]),
    "mindiesd_rf_token_order": (c_int, [c_p] + [c_int] * 5 + [c_p]),
    "mindiesd_fa_block_quant": (c_int, [c_p, c_p, c_p] + [c_int] * 5 + [c_ll] * 3 + [c_int, c_f, c_int, c_p]),
    "mindiesd_fa_rot_block_quant": (c_int, [c_p, c_p, c_p, c_p] + [c_int] * 5 + [c_ll] * 3 + [c_f, c_int, c_p]),
    "mindiesd_fp8_v_quant_workspace_size": (c_sz, [c_int, c_int]),
    "mindiesd_fp8_v_quant": (c_int, [c_p, c_p, c_p] + [c_int] * 5 + [c_ll] * 3 + [c_p, c_sz, c_p]),
    "mindiesd_fp8_v_quant_static_max_heads": (c_int, []),
    "mindiesd_fp8_v_quant_static": (c_int, [c_p, c_p, c_p] + [c_int] * 5 + [c_ll] * 3 + [c_p]),
    "mindiesd_fp8_attention_fwd": (c_int, [c_p] * 7 + [c_int] * 6 + [c_ll] * 3 + [c_f, c_int, c_p]),
    "mindiesd_mx_quant": (c_int, [c_p, c_p, c_p, c_int, c_ll, c_int, c_ll, c_p]),
    "mindiesd_mxfp8_gemm": (c_int, [c_p] * 6 + [c_int] * 5 + [c_p]),
}


def lib_path():
    return _LIB_PATH


def lib():
    """Load (once) and return the HIP library; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.isfile(_LIB_PATH):
            raise RuntimeError(
                f"mindiesd HIP library not found at {_LIB_PATH}; build it with "
                f"`python mindie-sd_amd/build.py` (there is no CPU fallback for fused ops)")
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed: {ERRORS.get(rc, 'error')} (code {rc})")


def stream_ptr(device=None):
    """The current HIP stream of ``device`` as an integer handle."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None and device is not None and device.index is not None:
        return raw(device.index)                      # (no Stream object: a microsecond less per call)
    return torch.cuda.current_stream(device).cuda_stream


class _Here:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_HERE = _Here()


def on_device(device):
    """Context that makes ``device`` the current one for the launch; nothing to do when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _HERE
    return torch.cuda.device(device)


DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1}
