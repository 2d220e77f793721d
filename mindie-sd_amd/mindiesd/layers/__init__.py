from . import _custom_ops  # noqa: F401  (declares torch.ops.mindiesd.*)
from .activation import get_activation_layer
from .flash_attn import attention_forward, attention_forward_varlen, sparse_attention

__all__ = ["attention_forward", "attention_forward_varlen", "get_activation_layer", "sparse_attention"]
