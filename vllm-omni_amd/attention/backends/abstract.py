"""Attention backend ABI: same classes, method names and argument meaning as the reference's
vllm_omni/diffusion/attention/backends/abstract.py:13-140."""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Generic, TypeVar

import torch


class AttentionBackend(ABC):
    """Class-level description of a backend; never instantiated (abstract.py:13-51)."""

    accept_output_buffer: bool = False

    @classmethod
    def supports_attention_mask(cls) -> bool:
        return False

    @staticmethod
    @abstractmethod
    def get_name() -> str: ...

    @staticmethod
    @abstractmethod
    def get_impl_cls() -> type["AttentionImpl"]: ...

    @staticmethod
    def get_metadata_cls() -> type["AttentionMetadata"]:
        return AttentionMetadata

    @staticmethod
    def get_builder_cls():
        raise NotImplementedError

    @staticmethod
    @abstractmethod
    def get_supported_head_sizes() -> list[int]: ...

    @classmethod
    def supports_head_size(cls, head_size: int) -> bool:
        sizes = cls.get_supported_head_sizes()
        return (not sizes) or head_size in sizes


@dataclass
class AttentionMetadata:
    """Per-call extras (abstract.py:54-66). ``attn_mask`` is a [B,Sk] key-padding mask; the joint_*
    fields carry a replicated text segment for sequence-parallel strategies and are unused on one GPU.
    ``output_split`` (not in the reference) asks the backend for two dense outputs, rows [0, s) and
    [s, Sq) of the joint sequence, instead of one tensor the caller would slice and copy.
    ``value_tail`` (not in the reference): the ``value`` argument then holds only the rows of the first
    keys and this tensor the rest, so a caller with the values of two streams in two buffers does not
    have to concatenate them.
    ``attn_mask_checked`` (not in the reference): the caller vouches that ``attn_mask`` is worth applying
    (it has already dropped an all-true mask, or accepts the masked kernel for one), so the backend skips
    its own all-true test, which costs a device-to-host synchronisation per call."""

    attn_mask: torch.Tensor | None = None
    joint_attn_mask: torch.Tensor | None = None
    joint_query: torch.Tensor | None = None
    joint_key: torch.Tensor | None = None
    joint_value: torch.Tensor | None = None
    joint_strategy: str = "front"
    output_split: int | None = None
    value_tail: torch.Tensor | None = None
    attn_mask_checked: bool = False


T = TypeVar("T", bound=AttentionMetadata)


class AttentionImpl(ABC, Generic[T]):
    """abstract.py:69-140. The reference's ``forward`` picks a per-platform method; with one platform
    here it is always ``forward_hip``, which each backend implements."""

    @abstractmethod
    def __init__(self, num_heads: int, head_size: int, softmax_scale: float, causal: bool = False,
                 num_kv_heads: int | None = None, prefix: str = "", **extra_impl_args) -> None: ...

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                attn_metadata: T | None = None) -> torch.Tensor:
        return self.forward_hip(query, key, value, attn_metadata)

    @abstractmethod
    def forward_hip(self, query, key, value, attn_metadata=None): ...
