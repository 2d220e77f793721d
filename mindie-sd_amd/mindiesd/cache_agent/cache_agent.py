"""CacheConfig / CacheAgent / AttentionCache with the reference's semantics (mindiesd/cache_agent/cache.py:17-57,
cache_agent.py:26-47, attention_cache.py:22-38).

A pipeline calls ``agent.apply(attention_fn, *args)`` once per transformer block and diffusion step, always in
the same order; the agent counts blocks and steps itself.  Inside the window ``step_start .. step_end`` the
attention of a block is computed only every ``step_interval``-th step and the stored result is returned in
between; after ``steps_count`` steps the counters and the store start over."""
from dataclasses import dataclass

from ..utils.exception import ConfigError, ParametersInvalid


@dataclass
class CacheConfig:
    method: str
    blocks_count: int
    steps_count: int
    step_start: int = 0
    step_interval: int = 1
    step_end: int = 10000
    block_start: int = 0
    block_end: int = 10000


class AttentionCache:
    def __init__(self, config: CacheConfig):
        self._config = config
        self._cur_step = 0
        self._cur_block = 0
        self._cache = [None] * config.blocks_count

    def apply(self, func, *args, **kwargs):
        res = self.apply_imp(func, *args, **kwargs)
        self._advance()
        return res

    def apply_imp(self, func, *args, **kwargs):
        cfg, step = self._config, self._cur_step
        in_window = cfg.step_start < step <= cfg.step_end
        if in_window and (step - cfg.step_start) % cfg.step_interval != 0:
            return self._cache[self._cur_block]                      # reuse
        attn = func(*args, **kwargs)
        if cfg.step_start <= step < cfg.step_end:                    # stored only while later steps may reuse it
            self._cache[self._cur_block] = attn
        return attn

    def _advance(self):
        self._cur_block += 1
        if self._cur_block == self._config.blocks_count:
            self._cur_block = 0
            self._cur_step += 1
            if self._cur_step == self._config.steps_count:           # one whole generation done
                self._cur_step = 0
                self._cache = [None] * self._config.blocks_count


CACHE_METHOD = {"attention_cache": AttentionCache}


class CacheAgent:
    def __init__(self, config: CacheConfig):
        self._config = config
        self._check_config()
        self._cache_method = CACHE_METHOD[config.method](config)

    def apply(self, function, *args, **kwargs):
        if not callable(function):
            raise ParametersInvalid("Input function must be callable.")
        cfg = self._config
        # settings under which nothing can ever be reused: call straight through, no counting
        if cfg.step_start >= cfg.steps_count or cfg.step_end == cfg.step_start:
            return function(*args, **kwargs)
        if cfg.block_start >= cfg.blocks_count or cfg.block_end == cfg.block_start:
            return function(*args, **kwargs)
        if cfg.step_interval == 1:
            return function(*args, **kwargs)
        return self._cache_method.apply(function, *args, **kwargs)

    def _check_config(self):
        cfg = self._config
        if cfg.method not in CACHE_METHOD:
            raise ConfigError(f"Method '{cfg.method}' is not supported, the list of support methods is "
                              f"{list(CACHE_METHOD.keys())}.")
        for name in ("blocks_count", "steps_count", "step_interval"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"The '{name}' in config must > 0, but got {getattr(cfg, name)}.")
        for name in ("step_start", "block_start"):
            if getattr(cfg, name) < 0:
                raise ConfigError(f"The '{name}' in config must >= 0, but got {getattr(cfg, name)}.")
        if cfg.step_end < cfg.step_start:
            raise ConfigError(f"The 'step_end' must >= 'step_start', but got {cfg.step_end} and {cfg.step_start}.")
        if cfg.block_end < cfg.block_start:
            raise ConfigError(f"The 'block_end' must >= 'block_start', but got {cfg.block_end} and {cfg.block_start}.")
