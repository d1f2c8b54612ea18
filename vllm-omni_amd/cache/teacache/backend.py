"""TeaCacheBackend: enable / refresh / is_enabled over a pipeline object that owns ``.transformer``
(vllm_omni/diffusion/cache/base.py:31-112, cache/teacache/backend.py:54-152)."""

from __future__ import annotations

from typing import Any

from ...hooks.base import HookRegistry
from .config import TeaCacheConfig
from .hook import TeaCacheHook, apply_teacache_hook


class TeaCacheBackend:
    def __init__(self, config: dict[str, Any] | TeaCacheConfig | None = None):
        self.config = config
        self.enabled = False

    def enable(self, pipeline: Any) -> None:
        transformer = pipeline.transformer
        cfg = self.config
        if not isinstance(cfg, TeaCacheConfig):
            kw = dict(cfg or {})
            kw.setdefault("transformer_type", transformer.__class__.__name__)
            cfg = TeaCacheConfig(**{k: v for k, v in kw.items()
                                    if k in ("rel_l1_thresh", "coefficients", "transformer_type")})
        self.config = cfg
        apply_teacache_hook(transformer, cfg)
        self.enabled = True

    def refresh(self, pipeline: Any, num_inference_steps: int, verbose: bool = True) -> None:
        """Forget all per-request state; called once before every request."""
        reg = getattr(pipeline.transformer, "_hook_registry", None)
        if reg is not None:
            reg.reset_hook(TeaCacheHook._HOOK_NAME)

    def is_enabled(self) -> bool:
        return self.enabled

    @staticmethod
    def hook_of(pipeline: Any) -> TeaCacheHook | None:
        reg = HookRegistry.get_or_create(pipeline.transformer)
        return reg.get_hook(TeaCacheHook._HOOK_NAME)
