from .flash_attn import attention_forward

__all__ = ["attention_forward"]
