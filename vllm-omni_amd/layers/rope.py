"""RotaryEmbedding: interleaved (GPT-J) or NeoX rotary on [B,S,H,D] with [S,rot/2] tables.

Interface of vllm_omni/diffusion/layers/rope.py:68-159; ``forward_hip`` runs the rotary stage of
the fused norm+rope kernel (no normalisation, q only) instead of flash-attn's triton kernel."""

from __future__ import annotations

import torch

from .. import kernels
from .._lib import ODIT_NORM_NONE
from .custom_op import CustomOp


class RotaryEmbedding(CustomOp):
    def __init__(self, is_neox_style: bool = False, ref_rounding: bool = False) -> None:
        super().__init__()
        self.is_neox_style = is_neox_style
        self.interleaved = not is_neox_style
        self.ref_rounding = ref_rounding

    def forward_hip(self, x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
        if cos.dim() == 3:  # (B,S,rot/2) -> first batch row, as rope.py:117-120
            cos, sin = cos[0], sin[0]
        if x.dim() != 4:
            raise ValueError("RotaryEmbedding expects x [B,S,H,D]")
        B, S, H, D = x.shape
        if x.stride(3) != 1 or x.stride(2) != D:
            x = x.contiguous()
        out = torch.empty((B, S, H, D), dtype=x.dtype, device=x.device)
        kernels.qknorm_rope(x, None, None, out, None, None, None, None, cos.float(), sin.float(),
                            norm_mode=ODIT_NORM_NONE, neox=self.is_neox_style,
                            ref_rounding=self.ref_rounding)
        return out
