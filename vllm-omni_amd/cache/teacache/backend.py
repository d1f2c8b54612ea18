"""TeaCacheBackend: enable / refresh / is_enabled over a pipeline object that owns ``.transformer``
(vllm_omni/diffusion/cache/base.py:31-112, cache/teacache/backend.py:54-152)."""

from __future__ import annotations

from typing import Any

from ...hooks.base import HookRegistry
from ..base import CacheBackend, DiffusionCacheConfig
from .config import TeaCacheConfig
from .hook import TeaCacheHook, apply_teacache_hook


class TeaCacheBackend(CacheBackend):
    def __init__(self, config: DiffusionCacheConfig | dict[str, Any] | TeaCacheConfig | None = None):
        """``config``: the reference's DiffusionCacheConfig (or a dict of its fields); a ready TeaCacheConfig is
        taken as it is. ``self.config`` keeps what was given, as in the reference."""
        if config is None or isinstance(config, dict):
            config = DiffusionCacheConfig.from_dict(config)
        super().__init__(config)

    def enable(self, pipeline: Any) -> None:
        transformer = pipeline.transformer
        cfg = self.config
        if not isinstance(cfg, TeaCacheConfig):
            try:
                cfg = TeaCacheConfig(transformer_type=transformer.__class__.__name__,
                                     rel_l1_thresh=cfg.rel_l1_thresh, coefficients=cfg.coefficients)
            except Exception as e:
                raise ValueError(f"Invalid TeaCache configuration: {e}. Expected keys: rel_l1_thresh, coefficients "
                                 "(optional); transformer_type comes from pipeline.transformer.__class__.__name__.") from e
        apply_teacache_hook(transformer, cfg)
        self.enabled = True

    def refresh(self, pipeline: Any, num_inference_steps: int, verbose: bool = True) -> None:
        """Forget all per-request state; called once before every request."""
        reg = getattr(pipeline.transformer, "_hook_registry", None)
        if reg is not None:
            reg.reset_hook(TeaCacheHook._HOOK_NAME)

    @staticmethod
    def hook_of(pipeline: Any) -> TeaCacheHook | None:
        reg = HookRegistry.get_or_create(pipeline.transformer)
        return reg.get_hook(TeaCacheHook._HOOK_NAME)
