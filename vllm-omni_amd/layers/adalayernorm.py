"""AdaLayerNorm: out = LayerNorm(x) * (1 + scale) + shift, returning (out, gate).

Same constructor, call signature and return tuple as
vllm_omni/diffusion/layers/adalayernorm.py:10-110; ``forward_hip`` is one launch of the fused
LayerNorm+modulate kernel instead of LayerNorm + mul + add."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import kernels
from .custom_op import CustomOp


class AdaLayerNorm(CustomOp):
    def __init__(self, hidden_size: int, elementwise_affine: bool = False, eps: float = 1e-6,
                 ref_rounding: bool = False) -> None:
        super().__init__()
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        self.hidden_size = hidden_size
        # parameter-less unless elementwise_affine, so state dicts line up with the reference's
        self.layernorm = nn.LayerNorm(hidden_size, elementwise_affine=elementwise_affine, eps=eps)
        self.ref_rounding = ref_rounding

    def preprocess(self, mod_params: torch.Tensor, index: torch.Tensor | None = None):
        """(shift, scale, gate) broadcastable against [B,L,C] (adalayernorm.py:23-60). Only ``gate``
        is materialised per token when ``index`` is given; shift/scale selection happens in-kernel."""
        shift, scale, gate = mod_params.chunk(3, dim=-1)
        if index is None:
            return shift.unsqueeze(1), scale.unsqueeze(1), gate.unsqueeze(1)
        nb = shift.size(0) // 2
        first = index.unsqueeze(-1) == 0

        def pick(t):
            return torch.where(first, t[:nb].unsqueeze(1), t[nb:].unsqueeze(1))

        return pick(shift), pick(scale), pick(gate)

    def forward_hip(self, x: torch.Tensor, mod_params: torch.Tensor, index: torch.Tensor | None = None):
        if x.shape[-1] != self.hidden_size:
            raise ValueError(f"expected last dim {self.hidden_size}, got {x.shape[-1]}")
        squeeze = x.dim() == 2
        x3 = x.unsqueeze(0) if squeeze else x
        shift, scale, gate = mod_params.chunk(3, dim=-1)
        lw = lb = None
        if self.elementwise_affine:
            lw = self.layernorm.weight.detach().float()
            lb = self.layernorm.bias.detach().float() if self.layernorm.bias is not None else None
        out = kernels.adaln_modulate(x3, shift, scale, eps=self.eps, index=index, ln_weight=lw,
                                     ln_bias=lb, ref_rounding=self.ref_rounding)
        if index is None:
            gate_result = gate.unsqueeze(1)
        else:
            nb = gate.size(0) // 2
            gate_result = torch.where(index.unsqueeze(-1) == 0, gate[:nb].unsqueeze(1), gate[nb:].unsqueeze(1))
        return (out.squeeze(0) if squeeze else out), gate_result
