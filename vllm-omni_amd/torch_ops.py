"""The per-layer kernels as ``torch.library`` custom ops (namespace ``omni_dit``).

The ctypes calls in ``kernels.py`` are opaque to ``torch.compile``: dynamo breaks the graph at each of
them. The reference compiles its repeated blocks region by region (vllm_omni/diffusion/compile.py:11-41,
``torch.compile(dynamic=True)`` unless ``enforce_eager``), so the drop-in layers call these ops instead:
each has a shape-only fake implementation, traces into one node and runs the same C-ABI entry point.
Only what the three per-layer interfaces need is wrapped (attention backend, AdaLayerNorm, RotaryEmbedding);
the fused block path of this package runs eager.
"""

from __future__ import annotations

import torch

from . import kernels
from ._lib import ODIT_NORM_NONE

_DEVICE = "cuda"  # torch's device type on ROCm builds


@torch.library.custom_op("omni_dit::attention", mutates_args=(), device_types=_DEVICE)
def attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale: float,
              key_mask: torch.Tensor | None = None) -> torch.Tensor:
    """softmax(q k^T * scale) v, q [B,Sq,H,D], k/v [B,Sk,Hkv,D], optional [B,Sk] key-padding mask."""
    return kernels.attn_fwd(query, key, value, scale, key_mask=key_mask)


@attention.register_fake
def _(query, key, value, scale, key_mask=None):
    return query.new_empty(query.shape)


@torch.library.custom_op("omni_dit::adaln_modulate", mutates_args=(), device_types=_DEVICE)
def adaln_modulate(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float,
                   index: torch.Tensor | None = None, ln_weight: torch.Tensor | None = None,
                   ln_bias: torch.Tensor | None = None) -> torch.Tensor:
    """LayerNorm(x) * (1 + scale) + shift for x [B,S,C]; shift/scale [B,C] ([2B,C] with ``index``)."""
    return kernels.adaln_modulate(x, shift, scale, eps=eps, index=index, ln_weight=ln_weight, ln_bias=ln_bias)


@adaln_modulate.register_fake
def _(x, shift, scale, eps, index=None, ln_weight=None, ln_bias=None):
    return x.new_empty(x.shape)


@torch.library.custom_op("omni_dit::rotary", mutates_args=(), device_types=_DEVICE)
def rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, neox: bool) -> torch.Tensor:
    """Rotary embedding of x [B,S,H,D] with float32 [S, rot/2] tables; interleaved pairs unless ``neox``."""
    B, S, H, D = x.shape
    if x.stride(3) != 1 or x.stride(2) != D:
        x = x.contiguous()
    out = torch.empty((B, S, H, D), dtype=x.dtype, device=x.device)
    kernels.qknorm_rope(x, None, None, out, None, None, None, None, cos, sin, norm_mode=ODIT_NORM_NONE, neox=neox)
    return out


@rotary.register_fake
def _(x, cos, sin, neox):
    return x.new_empty(x.shape)


# ------------------------------------------------------------------ bodies for the reference's classes
def adaln_forward_hip(self, x: torch.Tensor, mod_params: torch.Tensor, index: torch.Tensor | None = None):
    """``AdaLayerNorm.forward_hip`` (vllm_omni/diffusion/layers/adalayernorm.py:70-76): (out, gate). Uses
    only attributes the reference class has (``eps``, ``hidden_size``, ``layernorm``)."""
    squeeze = x.dim() == 2
    x3 = x.unsqueeze(0) if squeeze else x
    shift, scale, gate = mod_params.chunk(3, dim=-1)
    lw = getattr(self.layernorm, "weight", None)
    lb = getattr(self.layernorm, "bias", None)
    out = torch.ops.omni_dit.adaln_modulate(x3, shift, scale, float(self.eps), index,
                                            lw.float() if lw is not None else None,
                                            lb.float() if lb is not None else None)
    if index is None:
        gate_result = gate.unsqueeze(1)
    else:
        nb = gate.size(0) // 2
        gate_result = torch.where(index.unsqueeze(-1) == 0, gate[:nb].unsqueeze(1), gate[nb:].unsqueeze(1))
    return (out.squeeze(0) if squeeze else out), gate_result


def rope_forward_hip(self, x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``RotaryEmbedding.forward_hip`` (vllm_omni/diffusion/layers/rope.py:108-127): [B,S,rot/2] tables
    use their first batch row."""
    if cos.dim() == 3:
        cos, sin = cos[0], sin[0]
    return torch.ops.omni_dit.rotary(x, cos.float(), sin.float(), bool(self.is_neox_style))


def attention_forward_hip(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                          attn_metadata=None) -> torch.Tensor:
    """``AttentionImpl.forward_hip`` (vllm_omni/diffusion/attention/backends/abstract.py:86-140). The
    mask is handed to the kernel as it is: testing it for all-true would need a device-to-host copy,
    which a traced region cannot hold."""
    mask = getattr(attn_metadata, "attn_mask", None) if attn_metadata is not None else None
    if not self.kernel_takes_layer or not self.kernel_takes_mask(mask, query.shape[0], key.shape[1]):
        return self.sdpa.forward_hip(query, key, value, attn_metadata)  # torch's own op: traceable as it is
    return torch.ops.omni_dit.attention(query, key, value, float(self.softmax_scale), mask)
