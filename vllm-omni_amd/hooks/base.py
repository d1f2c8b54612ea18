"""Forward-interception hooks: ``HookRegistry`` wraps ``module.forward`` once and routes calls to
registered ``ModelHook`` objects; ``StateManager`` keeps one state object per named context.
Public surface of vllm_omni/diffusion/hooks/base.py:18-247."""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch.nn as nn


class BaseState:
    def reset(self) -> None:
        pass


class StateManager:
    """Lazily creates ``state_cls()`` per context name; ``reset`` forgets them all (base.py:25-42)."""

    def __init__(self, state_cls: Callable[[], BaseState]):
        self._state_cls = state_cls
        self._states: dict[str, BaseState] = {}
        self._context = "default"

    def set_context(self, name: str) -> None:
        self._context = name or "default"

    def get_state(self) -> BaseState:
        st = self._states.get(self._context)
        if st is None:
            st = self._states[self._context] = self._state_cls()
        return st

    def reset(self) -> None:
        self._states.clear()


class ModelHook:
    """Override ``pre_forward`` / ``post_forward`` to edit arguments or outputs, or ``new_forward``
    to replace the call altogether (base.py:45-122)."""

    def initialize_hook(self, module: nn.Module) -> nn.Module:
        return module

    def pre_forward(self, module: nn.Module, *args: Any, **kwargs: Any) -> tuple[tuple, dict]:
        return args, kwargs

    def post_forward(self, module: nn.Module, output: Any) -> Any:
        return output

    def new_forward(self, module: nn.Module, *args: Any, **kwargs: Any) -> Any:
        args, kwargs = self.pre_forward(module, *args, **kwargs)
        return self.post_forward(module, module._original_forward(*args, **kwargs))

    def reset_state(self, module: nn.Module) -> nn.Module:
        return module


class _WrappedForward:
    """Callable installed as ``module.forward`` (base.py:125-135)."""

    def __init__(self, module: nn.Module):
        self.module = module

    def __call__(self, *args: Any, **kwargs: Any):
        reg = getattr(self.module, "_hook_registry", None)
        if reg is None or not reg._hooks:
            return self.module._original_forward(*args, **kwargs)
        return reg.dispatch(*args, **kwargs)


class HookRegistry:
    def __init__(self, module: nn.Module):
        self.module = module
        self._hooks: dict[str, ModelHook] = {}

    @classmethod
    def get_or_create(cls, module: nn.Module) -> "HookRegistry":
        reg = getattr(module, "_hook_registry", None)
        if reg is None:
            reg = cls(module)
            module._hook_registry = reg
            if not hasattr(module, "_original_forward"):
                module._original_forward = module.forward
                module.forward = _WrappedForward(module)
        return reg

    def register_hook(self, name: str, hook: ModelHook) -> None:
        hook.initialize_hook(self.module)
        self._hooks[name] = hook

    def remove_hook(self, name: str) -> None:
        self._hooks.pop(name, None)

    def get_hook(self, name: str) -> ModelHook | None:
        return self._hooks.get(name)

    def dispatch(self, *args: Any, **kwargs: Any) -> Any:
        """One hook: its ``new_forward`` owns the call. Several: all ``pre_forward`` in name order,
        the original forward, then all ``post_forward`` in reverse (base.py:203-237)."""
        if not self._hooks:
            return self.module._original_forward(*args, **kwargs)
        if len(self._hooks) == 1:
            (hook,) = self._hooks.values()
            return hook.new_forward(self.module, *args, **kwargs)
        ordered = [self._hooks[k] for k in sorted(self._hooks)]
        for h in ordered:
            args, kwargs = h.pre_forward(self.module, *args, **kwargs)
        out = self.module._original_forward(*args, **kwargs)
        for h in reversed(ordered):
            out = h.post_forward(self.module, out)
        return out

    def reset_hook(self, name: str) -> None:
        hook = self._hooks.get(name)
        if hook is not None:
            hook.reset_state(self.module)
