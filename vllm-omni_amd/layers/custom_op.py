"""CustomOp base of this package's layers. The reference's ``CustomOp``
(vllm_omni/diffusion/layers/custom_op.py:9-53) picks one of five per-platform methods when the layer is
constructed; this package has one platform, so the method bound at construction is always
``forward_hip``, which every layer here implements on the gfx950 kernels. ``forward_native`` is kept as
the hook name the reference documents for a plain-torch version, and stays unimplemented: the torch
restatement of every op lives in the test oracle, not in the product."""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch.nn as nn


class CustomOp(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self._forward_method = self.dispatch_forward()

    def dispatch_forward(self) -> Callable:
        return self.forward_hip

    def forward(self, *args, **kwargs) -> Any:
        return self._forward_method(*args, **kwargs)

    def forward_hip(self, *args, **kwargs):
        raise NotImplementedError(f"{type(self).__name__} does not implement forward_hip")

    def forward_native(self, *args, **kwargs):
        raise NotImplementedError(f"{type(self).__name__} has no torch-native path in this package")
