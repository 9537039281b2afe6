from .base import HookStateT, NoOpWeightUpdateHook, WeightUpdateHook
from .hyperball import HyperballHook

__all__ = ["HookStateT", "HyperballHook", "NoOpWeightUpdateHook", "WeightUpdateHook"]
