"""Dispatch key and LRU cache of the attention front door (mindiesd/layers/flash_attn/common.py:20-61)."""
from collections import OrderedDict
from dataclasses import dataclass
from functools import wraps

import torch

attn_cache = OrderedDict()


def lru_cache_by_attn_param(maxsize=None):
    """Cache a function's result under ``attn_param.to_hash()`` with least-recently-used eviction."""
    def decorator(func):
        @wraps(func)
        def wrapper(attn_param, *args, **kwargs):
            key = attn_param.to_hash()
            if key in attn_cache:
                attn_cache.move_to_end(key)
                return attn_cache[key]
            value = func(attn_param, *args, **kwargs)
            attn_cache[key] = value
            if maxsize is not None and len(attn_cache) > maxsize:
                attn_cache.popitem(last=False)
            return value
        return wrapper
    return decorator


@dataclass
class AttentionParam:
    batch_size: int
    head_num: int
    head_dim: int
    q_seqlen: int
    kv_seqlen: int
    dtype: torch.dtype
    head_first: bool

    def to_str(self):
        return (f"batch_size:{self.batch_size}, head_num:{self.head_num}, head_dim:{self.head_dim}, "
                f"q_seqlen:{self.q_seqlen}, kv_seqlen:{self.kv_seqlen}, dtype:{self.dtype}, "
                f"head_first:{self.head_first}")

    def to_hash(self):
        return hash((self.batch_size, self.head_num, self.head_dim, self.q_seqlen, self.kv_seqlen,
                     self.dtype, self.head_first))
