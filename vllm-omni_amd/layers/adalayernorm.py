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


def adaln_pair(norm_a: AdaLayerNorm, x_a: torch.Tensor, mod_a: torch.Tensor,
               norm_b: AdaLayerNorm, x_b: torch.Tensor, mod_b: torch.Tensor):
    """``norm_a(x_a, mod_a)`` and ``norm_b(x_b, mod_b)`` (no index, no LayerNorm affine) in ONE launch: the
    two streams of a dual-stream block. Returns ((out_a, gate_a), (out_b, gate_b))."""
    if (norm_a.elementwise_affine or norm_b.elementwise_affine or norm_a.eps != norm_b.eps
            or norm_a.ref_rounding != norm_b.ref_rounding or x_a.dim() != 3 or x_b.dim() != 3):
        return norm_a(x_a, mod_a), norm_b(x_b, mod_b)
    shift_a, scale_a, gate_a = mod_a.chunk(3, dim=-1)
    shift_b, scale_b, gate_b = mod_b.chunk(3, dim=-1)
    out_a, out_b = kernels.adaln_modulate_pair((x_a, shift_a, scale_a), (x_b, shift_b, scale_b), eps=norm_a.eps,
                                               ref_rounding=norm_a.ref_rounding)
    return (out_a, gate_a.unsqueeze(1)), (out_b, gate_b.unsqueeze(1))
