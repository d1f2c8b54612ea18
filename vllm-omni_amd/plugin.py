"""Entry point that installs the gfx950 kernels into a vLLM-Omni process.

Declare it in the installing distribution as

    [project.entry-points."vllm_omni.general_plugins"]
    omni_dit = "vllm_omni_amd.plugin:register"

vLLM-Omni calls every function of that group once per process before models are built
(vllm_omni/plugins/__init__.py:61-74). That order matters: attention backends are resolved and cached when
the first ``Attention`` layer is constructed (vllm_omni/diffusion/attention/selector.py:54-85) and
``CustomOp`` layers capture their ``forward_hip`` in ``__init__``
(vllm_omni/diffusion/layers/custom_op.py:15-29).

What it installs:
  * ``CompiledHipFlashAttentionBackend`` under both names the ROCm platform can select — FLASH_ATTN (aiter
    present) and TORCH_SDPA (its fallback), vllm_omni/platforms/rocm/platform.py:31-67;
  * ``AdaLayerNorm.forward_hip`` and ``RotaryEmbedding.forward_hip``;
  * the Flux TeaCache extractor, for which the reference ships coefficients but no extractor
    (vllm_omni/diffusion/cache/teacache/extractors.py:575-615).
All three call ``torch.ops.omni_dit.*`` (see ``torch_ops``), so regional ``torch.compile`` keeps one graph.
The function is idempotent, as plugins may be loaded several times.
"""

from __future__ import annotations

from . import _lib, torch_ops
from .attention.backends.hip_flash import HipFlashAttentionBackend, HipFlashAttentionImpl

BACKEND_PATH = "vllm_omni_amd.plugin.CompiledHipFlashAttentionBackend"
OVERRIDDEN_BACKENDS = ("FLASH_ATTN", "TORCH_SDPA")


class CompiledHipFlashAttentionImpl(HipFlashAttentionImpl):
    """Same kernel as ``HipFlashAttentionImpl``, reached through the traceable custom op."""

    forward_hip = torch_ops.attention_forward_hip


class CompiledHipFlashAttentionBackend(HipFlashAttentionBackend):
    @staticmethod
    def get_impl_cls() -> type[CompiledHipFlashAttentionImpl]:
        return CompiledHipFlashAttentionImpl


def register() -> None:
    try:
        from vllm_omni.diffusion.attention.backends.registry import (
            DiffusionAttentionBackendEnum,
            register_diffusion_backend,
        )
        from vllm_omni.diffusion.cache.teacache.extractors import register_extractor
        from vllm_omni.diffusion.layers.adalayernorm import AdaLayerNorm
        from vllm_omni.diffusion.layers.rope import RotaryEmbedding
    except ImportError as e:
        raise ImportError("vllm_omni_amd.plugin.register() needs an importable vllm-omni install") from e
    _lib.load()  # a missing or stale kernel library must stop the worker here, not at the first block
    for name in OVERRIDDEN_BACKENDS:
        register_diffusion_backend(DiffusionAttentionBackendEnum[name], BACKEND_PATH)
    AdaLayerNorm.forward_hip = torch_ops.adaln_forward_hip
    RotaryEmbedding.forward_hip = torch_ops.rope_forward_hip
    from .cache.teacache.extractors import extract_flux_context

    register_extractor("FluxTransformer2DModel", extract_flux_context)
