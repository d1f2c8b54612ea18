"""Forward interception for one module, with the class and method names of
vllm_omni/diffusion/hooks/base.py:18-247 (``BaseState``, ``StateManager``, ``ModelHook``,
``HookRegistry``) so hooks written against the reference attach unchanged.

Design of this implementation: the registry does no work per call. Every change of the hook set
(``register_hook`` / ``remove_hook``) rebuilds ONE callable, the *route*, and ``module.forward`` is a
thin trampoline to the current route:

  * no hooks       -> the route IS the module's original bound forward;
  * one hook       -> the route is that hook's ``new_forward`` with the module bound in (the hook owns
                      the call and may never reach the original forward: that is how TeaCache skips);
  * several hooks  -> a pipeline: ``pre_forward`` of every hook in ascending name order, the original
                      forward, ``post_forward`` in descending name order.

The attributes ``module._original_forward`` and ``module._hook_registry`` are part of the interface:
hooks call the former, cache backends look up the latter.
"""

from __future__ import annotations

import functools
from collections.abc import Callable
from typing import Any

import torch.nn as nn

_DEFAULT_CONTEXT = "default"


class BaseState:
    """State container of a hook; ``reset`` returns it to its initial condition."""

    def reset(self) -> None:
        return None


class StateManager:
    """One lazily built ``state_cls()`` per context name (e.g. one per CFG branch); the current
    context is selected with ``set_context`` and an empty name selects ``"default"``."""

    def __init__(self, state_cls: Callable[[], BaseState]):
        self._factory = state_cls
        self._by_context: dict[str, BaseState] = {}
        self._current = _DEFAULT_CONTEXT

    def set_context(self, name: str) -> None:
        self._current = name if name else _DEFAULT_CONTEXT

    @property
    def current_context(self) -> str:
        return self._current

    def get_state(self) -> BaseState:
        try:
            return self._by_context[self._current]
        except KeyError:
            state = self._by_context[self._current] = self._factory()
            return state

    def reset(self) -> None:
        self._by_context = {}


class ModelHook:
    """A hook edits the call (``pre_forward``), its result (``post_forward``), or takes the whole call
    over (``new_forward``, whose default is pre -> original forward -> post)."""

    def initialize_hook(self, module: nn.Module) -> nn.Module:
        return module

    def pre_forward(self, module: nn.Module, *args: Any, **kwargs: Any) -> tuple[tuple, dict]:
        return args, kwargs

    def post_forward(self, module: nn.Module, output: Any) -> Any:
        return output

    def new_forward(self, module: nn.Module, *args: Any, **kwargs: Any) -> Any:
        call_args, call_kwargs = self.pre_forward(module, *args, **kwargs)
        return self.post_forward(module, module._original_forward(*call_args, **call_kwargs))

    def reset_state(self, module: nn.Module) -> nn.Module:
        return module


def _pipeline(module: nn.Module, hooks: list[ModelHook]) -> Callable[..., Any]:
    """Route for several hooks; ``hooks`` is already in ascending name order."""
    pres = [h.pre_forward for h in hooks]
    posts = [h.post_forward for h in hooks[::-1]]

    def route(*args: Any, **kwargs: Any) -> Any:
        for pre in pres:
            args, kwargs = pre(module, *args, **kwargs)
        result = module._original_forward(*args, **kwargs)
        for post in posts:
            result = post(module, result)
        return result

    return route


class HookRegistry:
    """The hooks of one module, by name. Obtain it with ``HookRegistry.get_or_create(module)``."""

    def __init__(self, module: nn.Module):
        self.module = module
        self._hooks: dict[str, ModelHook] = {}
        self._route: Callable[..., Any] | None = None  # None until the module's forward is captured

    # -- attachment ------------------------------------------------------------------------------
    @classmethod
    def get_or_create(cls, module: nn.Module) -> "HookRegistry":
        existing = getattr(module, "_hook_registry", None)
        if existing is not None:
            return existing
        registry = cls(module)
        if not hasattr(module, "_original_forward"):  # capture the forward exactly once per module
            module._original_forward = module.forward
            module.forward = registry._trampoline
        module._hook_registry = registry
        registry._rebuild()
        return registry

    def _trampoline(self, *args: Any, **kwargs: Any) -> Any:
        return self._route(*args, **kwargs)

    def _rebuild(self) -> None:
        module = self.module
        names = sorted(self._hooks)
        if not names:
            self._route = module._original_forward
        elif len(names) == 1:
            self._route = functools.partial(self._hooks[names[0]].new_forward, module)
        else:
            self._route = _pipeline(module, [self._hooks[n] for n in names])

    # -- hook set --------------------------------------------------------------------------------
    def register_hook(self, name: str, hook: ModelHook) -> None:
        hook.initialize_hook(self.module)
        self._hooks[name] = hook
        self._rebuild()

    def remove_hook(self, name: str) -> None:
        if self._hooks.pop(name, None) is not None:
            self._rebuild()

    def get_hook(self, name: str) -> ModelHook | None:
        return self._hooks.get(name)

    def reset_hook(self, name: str) -> None:
        hook = self._hooks.get(name)
        if hook is not None:
            hook.reset_state(self.module)

    def dispatch(self, *args: Any, **kwargs: Any) -> Any:
        """Run one call through the current route (what ``module(...)`` does)."""
        return self._route(*args, **kwargs)
