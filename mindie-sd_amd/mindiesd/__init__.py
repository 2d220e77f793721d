"""MI355X-native drop-in for the attention hot path of MindIE-SD (``import mindiesd``).

Public names follow mindiesd/__init__.py:13-44 for the part of the API this build covers."""
from .layers import attention_forward, attention_forward_varlen, sparse_attention
from .utils.exception import ParametersInvalid

__all__ = ["attention_forward", "attention_forward_varlen", "sparse_attention", "ParametersInvalid"]
