"""CacheContext and the extractor registry (vllm_omni/diffusion/cache/teacache/extractors.py:26-144,
575-650), plus extractors for the transformers built in this package."""

from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass
from typing import Any

import torch
import torch.nn as nn

from ... import kernels


@dataclass
class CacheContext:
    """What a model-specific extractor hands to the generic hook.

    modulated_input          tensor whose step-to-step change drives the skip decision
    hidden_states            stem output entering the blocks
    encoder_hidden_states    text stream for dual-stream models, else None
    temb                     timestep embedding
    run_transformer_blocks   () -> (hidden,) or (hidden, encoder) after all blocks
    postprocess              hidden -> model output
    run_transformer_blocks_rows  optional (rows: list[int]) -> same tuple for a subset of batch rows;
                             lets a CFG-batched call recompute only the rows whose branch must compute
    """

    modulated_input: torch.Tensor
    hidden_states: torch.Tensor
    encoder_hidden_states: torch.Tensor | None
    temb: torch.Tensor
    run_transformer_blocks: Callable[[], tuple[torch.Tensor, ...]]
    postprocess: Callable[[torch.Tensor], Any]
    extra_states: dict[str, Any] | None = None
    run_transformer_blocks_rows: Callable[[list[int]], tuple[torch.Tensor, ...]] | None = None

    def validate(self) -> None:
        for name in ("modulated_input", "hidden_states", "temb"):
            if not isinstance(getattr(self, name), torch.Tensor):
                raise TypeError(f"{name} must be torch.Tensor, got {type(getattr(self, name))}")
        if self.encoder_hidden_states is not None and not isinstance(self.encoder_hidden_states, torch.Tensor):
            raise TypeError(f"encoder_hidden_states must be torch.Tensor or None, got {type(self.encoder_hidden_states)}")
        for name in ("run_transformer_blocks", "postprocess"):
            if not callable(getattr(self, name)):
                raise TypeError(f"{name} must be callable, got {type(getattr(self, name))}")
        if self.modulated_input.shape[0] != self.hidden_states.shape[0]:
            raise ValueError(f"Batch size mismatch: modulated_input has batch size {self.modulated_input.shape[0]}, "
                             f"but hidden_states has {self.hidden_states.shape[0]}")
        if self.modulated_input.device != self.hidden_states.device:
            raise ValueError(f"Device mismatch: modulated_input on {self.modulated_input.device}, "
                             f"hidden_states on {self.hidden_states.device}")


def extract_qwen_context(module: nn.Module, hidden_states: torch.Tensor,
                         encoder_hidden_states: torch.Tensor, encoder_hidden_states_mask: torch.Tensor | None = None,
                         timestep: torch.Tensor | None = None, img_shapes=None, txt_seq_lens=None,
                         guidance: torch.Tensor | None = None, additional_t_cond=None,
                         attention_kwargs: dict[str, Any] | None = None, **kwargs: Any) -> CacheContext:
    """Qwen-Image: stem, then block 0's img_norm1 on the stem output is the decision tensor
    (extractors.py:147-279). ``module`` is this package's QwenImageTransformer2DModel."""
    if not hasattr(module, "transformer_blocks") or len(module.transformer_blocks) == 0:
        raise ValueError("Module must have transformer_blocks")
    if getattr(module, "zero_cond_t", False):
        # the reference's extractor passes no per-token index to the blocks either (extractors.py:245-254):
        # an editing model under it would silently be modulated wrongly, so refuse instead
        raise NotImplementedError("TeaCache has no extractor for the zero_cond_t (editing) variant")
    if guidance is not None:  # the reference hands it to a time embedding that takes none (extractors.py:199-203)
        raise TypeError("extract_qwen_context: the timestep embedding takes no guidance; pass guidance=None")
    img, txt, temb, rotary = module.prepare(hidden_states, encoder_hidden_states, timestep, img_shapes, txt_seq_lens,
                                            additional_t_cond)
    block0 = module.transformer_blocks[0]
    mod1 = block0.img_mod(temb).chunk(2, dim=-1)[0]
    shift, scale, _ = mod1.chunk(3, dim=-1)
    # The decision tensor is always rounded where the reference's torch ops round (one 50 MB elementwise pass
    # per step), whatever rounding the block stack itself runs with: skip/compute decisions then do not depend
    # on whether the model was built with fused GEMM epilogues.
    modulated = kernels.adaln_modulate(img, shift, scale, eps=block0.img_norm1.eps, ref_rounding=True)
    mask = encoder_hidden_states_mask
    return_dict = kwargs.get("return_dict", True)

    def run_rows(rows: list[int] | None):
        if rows is None:
            h, e, t, m = img, txt, temb, mask
        else:
            idx = torch.as_tensor(rows, device=img.device)
            h, e, t = img.index_select(0, idx), txt.index_select(0, idx), temb.index_select(0, idx)
            m = mask.index_select(0, idx) if mask is not None else None
        h, e = module.run_blocks(h, e, t, rotary, m, attention_kwargs)
        return (h, e)

    def postprocess(h):
        return module.finish(h, temb, return_dict=return_dict)

    return CacheContext(modulated_input=modulated, hidden_states=img, encoder_hidden_states=txt, temb=temb,
                        run_transformer_blocks=lambda: run_rows(None), postprocess=postprocess,
                        run_transformer_blocks_rows=run_rows)


def extract_flux_context(module: nn.Module, hidden_states: torch.Tensor,
                         encoder_hidden_states: torch.Tensor | None = None,
                         pooled_projections: torch.Tensor | None = None, timestep: torch.Tensor | None = None,
                         img_ids: torch.Tensor | None = None, txt_ids: torch.Tensor | None = None,
                         guidance: torch.Tensor | None = None,
                         joint_attention_kwargs: dict[str, Any] | None = None, **kwargs: Any) -> CacheContext:
    """Flux: stem, then block 0's norm1 (AdaLayerNormZero) on the x_embedder output is the decision
    tensor — the recipe the reference sketches for this model (extractors.py:580, 597-613) with the
    coefficients it already ships (config.py:11-17). ``module`` is this package's FluxTransformer2DModel."""
    if not hasattr(module, "transformer_blocks") or len(module.transformer_blocks) == 0:
        raise ValueError("Module must have transformer_blocks")
    if not hasattr(module, "prepare"):
        raise TypeError("extract_flux_context drives this package's FluxTransformer2DModel (prepare / run_blocks / "
                        f"finish stages); got {type(module).__module__}.{type(module).__name__}")
    img, txt, temb, rotary = module.prepare(hidden_states, encoder_hidden_states, pooled_projections, timestep,
                                            img_ids, txt_ids, guidance)
    norm1 = module.transformer_blocks[0].norm1
    shift, scale = norm1.linear(kernels.silu(temb)).chunk(6, dim=1)[:2]
    # reference rounding for the decision tensor, whatever the blocks run with (see extract_qwen_context)
    modulated = kernels.adaln_modulate(img, shift, scale, eps=norm1.eps, ref_rounding=True)
    return_dict = kwargs.get("return_dict", True)

    def run_rows(rows: list[int] | None):
        if rows is None:
            h, e, t = img, txt, temb
        else:
            idx = torch.as_tensor(rows, device=img.device)
            h, e, t = img.index_select(0, idx), txt.index_select(0, idx), temb.index_select(0, idx)
        return module.run_blocks(h, e, t, rotary, joint_attention_kwargs)

    def postprocess(h):
        return module.finish(h, temb, return_dict=return_dict)

    return CacheContext(modulated_input=modulated, hidden_states=img, encoder_hidden_states=txt, temb=temb,
                        run_transformer_blocks=lambda: run_rows(None), postprocess=postprocess,
                        run_transformer_blocks_rows=run_rows)


EXTRACTOR_REGISTRY: dict[str, Callable] = {
    "QwenImageTransformer2DModel": extract_qwen_context,
    "FluxTransformer2DModel": extract_flux_context,
}


def register_extractor(transformer_cls_name: str, extractor_fn: Callable) -> None:
    EXTRACTOR_REGISTRY[transformer_cls_name] = extractor_fn


def get_extractor(transformer_cls_name: str) -> Callable:
    try:
        return EXTRACTOR_REGISTRY[transformer_cls_name]
    except KeyError:
        raise ValueError(
            f"Unknown model type: '{transformer_cls_name}'. Available types: {list(EXTRACTOR_REGISTRY)}\n"
            "To add support for a new model, use register_extractor() or add to EXTRACTOR_REGISTRY.") from None
