"""CustomOp base: binds the platform's forward at construction, like
vllm_omni/diffusion/layers/custom_op.py:9-53. On this package's single platform that is always
``forward_hip``; ``forward_native`` stays an unimplemented hook (the torch restatement of every op
lives in the test oracle, not in the product)."""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch.nn as nn

from ..platforms import current_omni_platform


class CustomOp(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self._forward_method = self.dispatch_forward()

    def dispatch_forward(self) -> Callable:
        plat = current_omni_platform
        if plat.is_rocm():
            return self.forward_hip
        if plat.is_cuda():
            return self.forward_cuda
        if plat.is_npu():
            return self.forward_npu
        if plat.is_xpu():
            return self.forward_xpu
        return self.forward_native

    def forward(self, *args, **kwargs) -> Any:
        return self._forward_method(*args, **kwargs)

    def forward_native(self, *args, **kwargs):
        raise NotImplementedError(f"{type(self).__name__} has no torch-native path in this package")

    def forward_cuda(self, *args, **kwargs):
        raise NotImplementedError

    def forward_npu(self, *args, **kwargs):
        raise NotImplementedError

    def forward_xpu(self, *args, **kwargs):
        raise NotImplementedError

    def forward_hip(self, *args, **kwargs):
        return self.forward_cuda(*args, **kwargs)
