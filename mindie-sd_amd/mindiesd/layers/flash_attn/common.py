"""Dispatch key and LRU cache of the attention front door (mindiesd/layers/flash_attn/common.py:20-61).

``AttentionParam`` is the key of a dense-attention problem (what the kernel choice may depend on);
``lru_cache_by_attn_param`` memoises a chooser under that key.  ``attn_cache`` is the one table all decorated
functions share, as in the reference: its length and ``clear()`` are part of what callers rely on."""
import functools
from collections import OrderedDict
from typing import NamedTuple

import torch


class _RecentlyUsed(OrderedDict):
    """Mapping that keeps its entries in order of last use and forgets the oldest beyond ``limit``."""

    def lookup(self, key, make, limit):
        try:
            value = self[key]
        except KeyError:
            value = self[key] = make()
            while limit is not None and len(self) > limit:
                self.popitem(last=False)
        else:
            self.move_to_end(key)
        return value


attn_cache = _RecentlyUsed()


def lru_cache_by_attn_param(maxsize=None):
    """Decorator factory: ``f(attn_param, ...)`` is evaluated once per ``attn_param.to_hash()`` and then served
    from ``attn_cache`` (least recently used entries go first once the table holds more than ``maxsize``)."""
    def decorate(chooser):
        @functools.wraps(chooser)
        def cached(attn_param, *args, **kwargs):
            return attn_cache.lookup(attn_param.to_hash(), lambda: chooser(attn_param, *args, **kwargs), maxsize)
        return cached
    return decorate


class AttentionParam(NamedTuple):
    """Shape, dtype and layout of one dense attention call (fields and order of the reference's dataclass)."""
    batch_size: int
    head_num: int
    head_dim: int
    q_seqlen: int
    kv_seqlen: int
    dtype: torch.dtype
    head_first: bool

    def to_str(self):
        return ", ".join(f"{name}:{value}" for name, value in self._asdict().items())

    def to_hash(self):
        return hash(tuple(self))
