"""torch SDPA backend: the reference keeps it as the float32 route of every Attention layer
(vllm_omni/diffusion/attention/layer.py:50-57, 134-143; backends/sdpa.py:38-92). It runs on whatever
device the tensors are on; 16-bit inputs never come here unless a user selects it explicitly."""

from __future__ import annotations

import torch

from .abstract import AttentionBackend, AttentionImpl, AttentionMetadata


class SDPABackend(AttentionBackend):
    accept_output_buffer: bool = True

    @classmethod
    def supports_attention_mask(cls) -> bool:
        return True

    @staticmethod
    def get_name() -> str:
        return "SDPA"

    @staticmethod
    def get_impl_cls() -> type["SDPAImpl"]:
        return SDPAImpl

    @staticmethod
    def get_supported_head_sizes() -> list[int]:
        return []  # any


class SDPAImpl(AttentionImpl):
    def __init__(self, num_heads: int, head_size: int, softmax_scale: float, causal: bool = False,
                 num_kv_heads: int | None = None, prefix: str = "", **extra_impl_args) -> None:
        self.causal = causal
        self.softmax_scale = softmax_scale

    def forward_hip(self, query, key, value, attn_metadata: AttentionMetadata | None = None):
        if attn_metadata is not None and attn_metadata.value_tail is not None:
            value = torch.cat([value, attn_metadata.value_tail], dim=1)
        q, k, v = (t.transpose(1, 2) for t in (query, key, value))
        mask = attn_metadata.attn_mask if attn_metadata else None
        if mask is not None and mask.dim() == 2:  # [B,Sk] key padding -> broadcastable boolean
            mask = mask.to(torch.bool)[:, None, None, :]
        out = torch.nn.functional.scaled_dot_product_attention(
            q, k, v, attn_mask=mask, dropout_p=0.0, is_causal=self.causal, scale=self.softmax_scale,
            enable_gqa=k.shape[1] != q.shape[1])
        out = out.transpose(1, 2)
        split = attn_metadata.output_split if attn_metadata else None
        if split is not None:
            return out[:, :split].contiguous(), out[:, split:].contiguous()
        return out
