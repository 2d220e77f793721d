from .attention_forward import attention_forward
from .attention_func import attention_math

__all__ = ["attention_forward", "attention_math"]
