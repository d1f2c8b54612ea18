from .base import BaseState, HookRegistry, ModelHook, StateManager

__all__ = ["BaseState", "HookRegistry", "ModelHook", "StateManager"]
