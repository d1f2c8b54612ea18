"""The MI355X attention backend: AttentionImpl.forward_hip -> odit_attn_fwd (hand-written gfx950
flash attention). Takes the place of FlashAttentionBackend (aiter / flash-attn,
vllm_omni/diffusion/attention/backends/flash_attn.py:25-115) and of SDPABackend for 16-bit inputs."""

from __future__ import annotations

import torch

from ... import kernels
from .abstract import AttentionBackend, AttentionImpl, AttentionMetadata


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
        return [64, 128]


class HipFlashAttentionImpl(AttentionImpl):
    def __init__(self, num_heads: int, head_size: int, softmax_scale: float, causal: bool = False,
                 num_kv_heads: int | None = None, prefix: str = "", **extra_impl_args) -> None:
        if causal:
            raise NotImplementedError("HipFlashAttentionImpl is non-causal (DiT joint attention)")
        if head_size not in HipFlashAttentionBackend.get_supported_head_sizes():
            raise ValueError(f"head_size {head_size} not supported; supported: 64, 128")
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        self.head_size = head_size
        self.softmax_scale = float(softmax_scale)
        self.causal = False

    def forward_hip(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                    attn_metadata: AttentionMetadata | None = None) -> torch.Tensor:
        """q [B,Sq,H,D], k/v [B,Sk,Hkv,D] -> [B,Sq,H,D]. A [B,Sk] ``attn_mask`` excludes keys; an
        all-true mask is dropped like the reference does (flash_attn.py:80-84) unless
        ``attn_metadata.attn_mask_checked`` says the caller has seen to that (the test synchronises). With
        ``attn_metadata.output_split`` = s the result is the pair (out[:, :s], out[:, s:]), both dense;
        with ``attn_metadata.value_tail`` the values are [value; value_tail] along the keys, read in place."""
        mask = attn_metadata.attn_mask if attn_metadata is not None else None
        if mask is not None:
            if mask.dim() != 2:
                raise ValueError("HipFlashAttentionImpl takes a [B,Sk] key-padding mask")
            if not attn_metadata.attn_mask_checked and bool(torch.all(mask != 0)):
                mask = None
        split = attn_metadata.output_split if attn_metadata is not None else None
        v_tail = attn_metadata.value_tail if attn_metadata is not None else None
        if v_tail is not None:
            value = (value, v_tail)
        return kernels.attn_fwd(query, key, value, self.softmax_scale, key_mask=mask, split=split)
