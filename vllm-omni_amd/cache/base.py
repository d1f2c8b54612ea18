"""Cache-backend interface and its configuration object (vllm_omni/diffusion/cache/base.py:31-102,
vllm_omni/diffusion/data.py:129-200). Only the TeaCache fields of the configuration are kept: the other
backend of the reference (cache-dit, a third-party library) is not part of this package."""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass, fields
from typing import Any


@dataclass
class DiffusionCacheConfig:
    """``rel_l1_thresh``: accumulated-change threshold (0.2 = the reference's default); ``coefficients``:
    five polynomial coefficients, None = the table entry of the transformer class."""

    rel_l1_thresh: float = 0.2
    coefficients: list[float] | None = None

    @classmethod
    def from_dict(cls, data: dict[str, Any] | None) -> "DiffusionCacheConfig":
        """Keys this package has no field for (the cache-dit parameters) are ignored."""
        known = {f.name for f in fields(cls)}
        return cls(**{k: v for k, v in (data or {}).items() if k in known})


class CacheBackend(ABC):
    def __init__(self, config: DiffusionCacheConfig):
        self.config = config
        self.enabled = False

    @abstractmethod
    def enable(self, pipeline: Any) -> None: ...

    @abstractmethod
    def refresh(self, pipeline: Any, num_inference_steps: int, verbose: bool = True) -> None: ...

    def is_enabled(self) -> bool:
        return self.enabled

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}(config={self.config})"
