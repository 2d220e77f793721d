"""Operator registration under the ``mindiesd::`` namespace.

The reference loads a C++ ``TORCH_LIBRARY(mindiesd, ...)`` plugin (csrc/plugin/register_ops.cpp:25-82,
mindiesd/layers/register_ops.py:24-48) and attaches fake (meta) implementations to its ops
(:90-128).  Here the schemas are declared from Python with ``torch.library``; the device
implementations (registered for the CUDA/HIP dispatch key) call the C ABI of
``plugin/libmindiesd_hip.so`` through ctypes.  Registration does not need a GPU, so a CPU-only import
works; calling an op without the library or a GPU raises.
"""
import torch

NAMESPACE = "mindiesd"
_lib_def = torch.library.Library(NAMESPACE, "FRAGMENT")
_defined = set()


def define_op(name, schema):
    """Declare ``mindiesd::name`` once per process."""
    if name in _defined:
        return
    _lib_def.define(f"{name}{schema}")
    _defined.add(name)


def register_device_impl(name):
    """Decorator: implementation for GPU tensors."""
    def decorator(func):
        _lib_def.impl(name, func, "CUDA")
        return func
    return decorator


def register_mindie_fake_op(name):
    """Decorator: shape/dtype-only implementation used by torch.compile / meta tensors."""
    def decorator(func):
        torch.library.register_fake(f"{NAMESPACE}::{name}")(func)
        return func
    return decorator
