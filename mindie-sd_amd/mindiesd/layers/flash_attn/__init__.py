from .attention_forward import attention_forward
from .attention_forward_varlen import attention_forward_varlen
from .attention_func import attention_math
from .sparse_flash_attn import sparse_attention
from .rainfusion import bsa_sparse_attention_v3

__all__ = ["attention_forward", "attention_forward_varlen", "attention_math", "sparse_attention", "bsa_sparse_attention_v3"]
