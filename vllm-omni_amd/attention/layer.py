"""Attention layer (vllm_omni/diffusion/attention/layer.py:26-152) for one GPU: no parallel
strategy (pre/post attention are the identity, parallel/base.py:61-82), float32 inputs are routed to
the SDPA implementation exactly as the reference does, everything else goes to the selected backend."""

from __future__ import annotations

import logging

import torch
import torch.nn as nn

from .backends.abstract import AttentionMetadata
from .backends.sdpa import SDPABackend
from .selector import get_attn_backend

logger = logging.getLogger(__name__)
_warned_fp32 = False


class Attention(nn.Module):
    def __init__(self, num_heads: int, head_size: int, causal: bool, softmax_scale: float,
                 num_kv_heads: int | None = None, prefix: str = "", scatter_idx: int = 2,
                 gather_idx: int = 1, use_sync: bool = False):
        super().__init__()
        self.attn_backend = get_attn_backend(-1)
        self.attn_impl_cls = self.attn_backend.get_impl_cls()
        kw = dict(num_heads=num_heads, head_size=head_size, softmax_scale=softmax_scale, causal=causal,
                  num_kv_heads=num_kv_heads)
        self.attention = self.attn_impl_cls(**kw)
        self.sdpa_fallback = SDPABackend.get_impl_cls()(**kw)
        self.softmax_scale = softmax_scale
        self.causal = causal
        self.scatter_idx, self.gather_idx, self.use_sync = scatter_idx, gather_idx, use_sync

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                attn_metadata: AttentionMetadata | None = None) -> torch.Tensor:
        return self._run_local_attention(query, key, value, attn_metadata)

    def _run_local_attention(self, query, key, value, attn_metadata):
        global _warned_fp32
        if query.dtype == torch.float32:
            if not _warned_fp32:
                logger.warning("Only SDPA supports float32; using it instead of %s", type(self.attention).__name__)
                _warned_fp32 = True
            return self.sdpa_fallback.forward(query, key, value, attn_metadata)
        return self.attention.forward(query, key, value, attn_metadata)
