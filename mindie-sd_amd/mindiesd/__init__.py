"""MI355X-native drop-in for the attention hot path of MindIE-SD (``import mindiesd``).

Public names follow mindiesd/__init__.py:13-44 for the part of the API this build covers."""
from .cache_agent import CacheAgent, CacheConfig
from .layers import attention_forward, attention_forward_varlen, get_activation_layer, sparse_attention
from .quantization import quantize
from .utils.exception import ConfigError, ParametersInvalid

__all__ = ["CacheConfig", "CacheAgent", "attention_forward", "attention_forward_varlen", "get_activation_layer",
           "quantize", "sparse_attention", "ParametersInvalid", "ConfigError"]
