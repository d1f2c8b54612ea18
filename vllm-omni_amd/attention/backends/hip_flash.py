"""The MI355X attention backend: AttentionImpl.forward_hip -> odit_attn_fwd (hand-written gfx950
flash attention). Takes the place of FlashAttentionBackend (aiter / flash-attn,
vllm_omni/diffusion/attention/backends/flash_attn.py:25-115) and of SDPABackend for 16-bit inputs.

The kernel is the non-causal joint attention of the DiT blocks: head sizes 64 and 128, an optional [B,Sk]
key-padding mask. What the backends it replaces also take (vllm_omni/diffusion/attention/backends/sdpa.py:73-92:
causal attention, any head size, masks of any shape that broadcasts against [B,H,Sq,Sk], boolean or additive)
goes to this package's SDPA backend, the way float32 inputs already do (attention/layer.py), so a model outside
the DiT families keeps running when this backend is installed under the names FLASH_ATTN and TORCH_SDPA."""

from __future__ import annotations

import torch

from ... import kernels
from .abstract import AttentionBackend, AttentionImpl, AttentionMetadata
from .sdpa import SDPAImpl

KERNEL_HEAD_SIZES = (64, 128)


class HipFlashAttentionBackend(AttentionBackend):
    accept_output_buffer: bool = False

    @classmethod
    def supports_attention_mask(cls) -> bool:
        return True

    @staticmethod
    def get_name() -> str:
        return "HIP_FLASH_ATTN"

    @staticmethod
    def get_impl_cls() -> type["HipFlashAttentionImpl"]:
        return HipFlashAttentionImpl

    @staticmethod
    def get_supported_head_sizes() -> list[int]:
        """Head sizes the kernel takes; other sizes are served through the SDPA route of the impl."""
        return list(KERNEL_HEAD_SIZES)


class HipFlashAttentionImpl(AttentionImpl):
    def __init__(self, num_heads: int, head_size: int, softmax_scale: float, causal: bool = False,
                 num_kv_heads: int | None = None, prefix: str = "", **extra_impl_args) -> None:
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        self.head_size = head_size
        self.softmax_scale = float(softmax_scale)
        self.causal = bool(causal)
        # the route for what the kernel does not take, chosen here (causal, head size) or per call (mask shape)
        self.sdpa = SDPAImpl(num_heads=num_heads, head_size=head_size, softmax_scale=softmax_scale, causal=causal,
                             num_kv_heads=num_kv_heads, prefix=prefix, **extra_impl_args)
        self.kernel_takes_layer = not self.causal and head_size in KERNEL_HEAD_SIZES

    @staticmethod
    def kernel_takes_mask(mask: torch.Tensor | None, batch: int, keys: int) -> bool:
        """None, or a [B,Sk] key-padding mask (boolean or 0/1 integers). Everything else (additive float masks,
        [B,1,1,Sk], [B,H,Sq,Sk], [Sq,Sk]) is SDPA's."""
        return mask is None or (mask.dim() == 2 and tuple(mask.shape) == (batch, keys) and not mask.is_floating_point())

    def forward_hip(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                    attn_metadata: AttentionMetadata | None = None) -> torch.Tensor:
        """q [B,Sq,H,D], k/v [B,Sk,Hkv,D] -> [B,Sq,H,D]. A [B,Sk] ``attn_mask`` excludes keys; an
        all-true mask is dropped like the reference does (flash_attn.py:80-84) unless
        ``attn_metadata.attn_mask_checked`` says the caller has seen to that (the test synchronises). With
        ``attn_metadata.output_split`` = s the result is the pair (out[:, :s], out[:, s:]), both dense;
        with ``attn_metadata.value_tail`` the values are [value; value_tail] along the keys, read in place."""
        mask = attn_metadata.attn_mask if attn_metadata is not None else None
        if not self.kernel_takes_layer or not self.kernel_takes_mask(mask, query.shape[0], key.shape[1]):
            return self.sdpa.forward_hip(query, key, value, attn_metadata)
        if mask is not None:
            if not attn_metadata.attn_mask_checked and bool(torch.all(mask != 0)):
                mask = None
        split = attn_metadata.output_split if attn_metadata is not None else None
        v_tail = attn_metadata.value_tail if attn_metadata is not None else None
        if v_tail is not None:
            value = (value, v_tail)
        return kernels.attn_fwd(query, key, value, self.softmax_scale, key_mask=mask, split=split)
