"""Backend registry: the closed enum of backend names plus run-time overrides, as in
vllm_omni/diffusion/attention/backends/registry.py:23-152. The defaults of FLASH_ATTN and TORCH_SDPA
point at this package's classes; ``register_diffusion_backend`` re-points a name at another class."""

from __future__ import annotations

import importlib
from collections.abc import Callable
from enum import Enum, EnumMeta


class _EnumMeta(EnumMeta):
    def __getitem__(cls, name: str):
        try:
            return super().__getitem__(name)
        except KeyError:
            valid = ", ".join(cls.__members__)
            raise ValueError(f"Unknown diffusion attention backend: '{name}'. Valid options are: {valid}") from None


_PKG = __name__.rsplit(".", 1)[0]


class DiffusionAttentionBackendEnum(Enum, metaclass=_EnumMeta):
    FLASH_ATTN = f"{_PKG}.hip_flash.HipFlashAttentionBackend"
    TORCH_SDPA = f"{_PKG}.sdpa.SDPABackend"
    SAGE_ATTN = ""  # int8 attention: no kernel in this package; must be registered to be used

    def get_path(self, include_classname: bool = True) -> str:
        path = _OVERRIDES.get(self, self.value)
        if not path:
            raise ValueError(
                f"Backend {self.name} must be registered before use. Use "
                f"register_diffusion_backend(DiffusionAttentionBackendEnum.{self.name}, 'your.module.YourClass')")
        return path if include_classname else path.rsplit(".", 1)[0]

    def get_class(self):
        mod, _, cls = self.get_path().rpartition(".")
        return getattr(importlib.import_module(mod), cls)

    def is_overridden(self) -> bool:
        return self in _OVERRIDES

    def clear_override(self) -> None:
        _OVERRIDES.pop(self, None)


_OVERRIDES: dict[DiffusionAttentionBackendEnum, str] = {}


def register_diffusion_backend(backend: DiffusionAttentionBackendEnum,
                               class_path: str | None = None) -> Callable[[type], type]:
    """Direct form ``register_diffusion_backend(E.X, "pkg.mod.Cls")`` or decorator form."""
    if class_path is not None:
        _OVERRIDES[backend] = class_path
        return lambda cls: cls

    def deco(cls: type) -> type:
        _OVERRIDES[backend] = f"{cls.__module__}.{cls.__qualname__}"
        return cls

    return deco
