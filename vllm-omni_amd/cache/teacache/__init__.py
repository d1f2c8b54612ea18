from .backend import TeaCacheBackend
from .config import TeaCacheConfig
from .extractors import CacheContext, get_extractor, register_extractor
from .hook import TeaCacheHook, apply_teacache_hook
from .state import TeaCacheState

__all__ = ["CacheContext", "TeaCacheBackend", "TeaCacheConfig", "TeaCacheHook", "TeaCacheState",
           "apply_teacache_hook", "get_extractor", "register_extractor"]
