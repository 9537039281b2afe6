"""Hook protocol around the final ``p.add_(update, alpha=-lr)`` (reference: weight_update_hooks/base.py:26-59)."""

from __future__ import annotations

from typing import Optional, Protocol, TypeVar

import torch


__all__ = ["NoOpWeightUpdateHook", "WeightUpdateHook", "HookStateT"]

HookStateT = TypeVar("HookStateT", bound=Optional[torch.Tensor])


class WeightUpdateHook(Protocol[HookStateT]):
    """``pre_weight_update_inplace`` runs right before the update and may return state that
    ``post_weight_update_inplace`` receives right after it."""

    def pre_weight_update_inplace(self, p: torch.Tensor, update: torch.Tensor) -> HookStateT: ...

    def post_weight_update_inplace(self, p: torch.Tensor, pre_update_state: HookStateT) -> None: ...


class NoOpWeightUpdateHook:
    """The default hook: does nothing on either side of the update."""

    def pre_weight_update_inplace(self, p: torch.Tensor, update: torch.Tensor) -> None:
        return None

    def post_weight_update_inplace(self, p: torch.Tensor, pre_update_state: None) -> None:
        return None
