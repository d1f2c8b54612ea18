from .backends.abstract import AttentionBackend, AttentionImpl, AttentionMetadata
from .layer import Attention
from .selector import get_attn_backend

__all__ = ["Attention", "AttentionBackend", "AttentionImpl", "AttentionMetadata", "get_attn_backend"]
