"""Per-CFG-branch TeaCache state (vllm_omni/diffusion/cache/teacache/state.py:13-38)."""

from __future__ import annotations

import torch

from ...hooks.base import BaseState


class TeaCacheState(BaseState):
    def __init__(self) -> None:
        self.reset()

    def reset(self) -> None:
        self.cnt = 0
        self.accumulated_rel_l1_distance = 0.0
        self.previous_modulated_input: torch.Tensor | None = None
        self.previous_residual: torch.Tensor | None = None
        self.previous_residual_encoder: torch.Tensor | None = None
