"""Platform object the dispatching classes consult.

Mirrors the queries the reference makes of ``current_omni_platform``
(vllm_omni/platforms/__init__.py, platforms/rocm/platform.py:31-67). This package has exactly one
platform: ROCm on gfx950, so ``CustomOp`` and ``AttentionImpl`` always run their ``forward_hip``.
"""

from __future__ import annotations


class RocmGfx950Platform:
    device_name = "rocm"
    device_type = "cuda"  # torch device string on ROCm builds
    arch = "gfx950"

    def is_rocm(self) -> bool:
        return True

    def get_diffusion_attn_backend_cls(self, selected_backend: str | None, head_size: int) -> str:
        """Qualified class name of the attention backend (platforms/rocm/platform.py:31-67 picks
        FLASH_ATTN when aiter is importable, else TORCH_SDPA; here both names resolve through the
        registry, whose overrides point at the HIP backend)."""
        from .attention.backends.registry import DiffusionAttentionBackendEnum

        name = (selected_backend or "FLASH_ATTN").upper()
        return DiffusionAttentionBackendEnum[name].get_path()

    def __repr__(self) -> str:
        return "RocmGfx950Platform()"


current_omni_platform = RocmGfx950Platform()
