"""Backend selection (vllm_omni/diffusion/attention/selector.py:54-85): an explicit name from the
DIFFUSION_ATTENTION_BACKEND environment variable wins, otherwise the platform chooses; the result
is cached per head size, so overrides must be registered before the first Attention layer is built."""

from __future__ import annotations

import importlib
import os
from functools import cache

from ..platforms import current_omni_platform
from .backends.abstract import AttentionBackend


@cache
def get_attn_backend(head_size: int) -> type[AttentionBackend]:
    selected = os.environ.get("DIFFUSION_ATTENTION_BACKEND")
    path = current_omni_platform.get_diffusion_attn_backend_cls(selected, head_size)
    mod, _, cls = path.rpartition(".")
    return getattr(importlib.import_module(mod), cls)
