"""RMSNorm over the last axis, standing in for vllm.model_executor.layers.layernorm.RMSNorm at the
reference's call sites (qwen_image_transformer.py:505-506, 543-544, 918): fp32 statistics, weight
multiply, one pass. Rows up to 8192 16-bit elements (one wavefront keeps the row in registers)."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import kernels
from .._lib import ODIT_NORM_HEAD, ODIT_NORM_ROW
from .custom_op import CustomOp


class RMSNorm(CustomOp):
    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.hidden_size = hidden_size
        self.variance_epsilon = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        n = self.hidden_size
        if x.shape[-1] != n:
            raise ValueError(f"expected last dim {n}, got {x.shape[-1]}")
        epv = 4 if x.dtype == torch.float32 else 8
        lanes = n // epv
        if n % epv == 0 and lanes <= 64 and lanes & (lanes - 1) == 0:
            heads, hd, mode = 1, n, ODIT_NORM_HEAD  # the row is one "head"
        else:
            # whole-row statistics; the (heads, hd) split only has to tile the row in 16-byte vectors
            hd = next((d for d in (128, 64, 32, 16, 8) if n % d == 0), None)
            if hd is None:
                raise ValueError(f"RMSNorm width {n} must be a multiple of 8")
            heads, mode = n // hd, ODIT_NORM_ROW
        x2 = x.reshape(1, -1, heads, hd)
        if x2.stride(3) != 1 or x2.stride(2) != hd:
            x2 = x2.contiguous()
        out = torch.empty((1, x2.shape[1], heads, hd), dtype=x.dtype, device=x.device)
        w = self.weight.detach()
        if w.dtype != x.dtype:
            w = w.float()
        kernels.qknorm_rope(x2, None, None, out, None, None, w, None, None, None,
                            eps=self.variance_epsilon, norm_mode=mode)
        return out.reshape(x.shape)
