"""get_cache_backend (vllm_omni/diffusion/cache/selector.py:9-38)."""

from __future__ import annotations

from typing import Any

from .base import CacheBackend, DiffusionCacheConfig


def get_cache_backend(cache_backend: str | None, cache_config: Any) -> CacheBackend | None:
    if cache_backend is None or cache_backend == "none":
        return None
    if isinstance(cache_config, dict):
        cache_config = DiffusionCacheConfig.from_dict(cache_config)
    if cache_backend == "tea_cache":
        from .teacache.backend import TeaCacheBackend

        return TeaCacheBackend(cache_config)
    if cache_backend == "cache_dit":
        raise NotImplementedError("the cache_dit backend wraps a third-party library and is not part of this package")
    raise ValueError(f"Unsupported cache backend: {cache_backend}. Supported: 'tea_cache'")
