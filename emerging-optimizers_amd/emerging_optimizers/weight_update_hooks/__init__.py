from .base import HookStateT, NoOpWeightUpdateHook, WeightUpdateHook

__all__ = ["HookStateT", "NoOpWeightUpdateHook", "WeightUpdateHook"]
