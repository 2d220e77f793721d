"""Device probe (counterpart of mindiesd/utils/utils.py:17 ``is_npu_available``)."""
import torch


def is_gpu_available():
    try:
        return torch.cuda.is_available() and torch.version.hip is not None
    except Exception:  # pragma: no cover - defensive: a broken driver must not break import
        return False
