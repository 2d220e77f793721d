"""Step-level reuse of attention results across diffusion steps (mindiesd/cache_agent): the caller of the attention
functions of this build.  Only the 'attention_cache' method is part of it."""
from .cache_agent import AttentionCache, CacheAgent, CacheConfig

__all__ = ["AttentionCache", "CacheAgent", "CacheConfig"]
