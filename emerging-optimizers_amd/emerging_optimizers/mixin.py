"""Weight-decay flavours shared by the optimizers (reference: emerging_optimizers/mixin.py:23-56)."""

from __future__ import annotations

from typing import Literal

import torch


WeightDecayT = Literal["decoupled", "independent", "l2", "palm"]


class WeightDecayMixin:
    """Adds ``_apply_weight_decay_inplace``; the flavour is read from ``self.weight_decay_method`` ("l2" if unset).

    ========== ==================================
    method      effect
    ========== ==================================
    decoupled   ``p -= wd * lr * p``
    independent ``p -= wd * p``
    l2          ``grad += wd * p``
    palm        ``p -= wd * lr**2 * p``
    ========== ==================================
    """

    def _apply_weight_decay_inplace(self, p: torch.Tensor, grad: torch.Tensor, lr: float, weight_decay: float) -> None:
        if weight_decay == 0.0:
            return
        method = getattr(self, "weight_decay_method", "l2")
        if method == "l2":
            grad.add_(p, alpha=weight_decay)
            return
        shrink = {
            "decoupled": weight_decay * lr,
            "independent": weight_decay,
            "palm": weight_decay * lr * lr,
        }.get(method)
        if shrink is None:
            raise ValueError(f"Invalid weight decay method: {method}")
        p.add_(p, alpha=-shrink)

    def _apply_weight_decay_foreach_inplace(
        self, params: list[torch.Tensor], grads: list[torch.Tensor], lr: float, weight_decay: float
    ) -> None:
        """The same update for a list of parameters, in one multi-tensor launch (element for element identical)."""
        if weight_decay == 0.0 or not params:
            return
        method = getattr(self, "weight_decay_method", "l2")
        if method == "l2":
            torch._foreach_add_(grads, params, alpha=weight_decay)
            return
        shrink = {
            "decoupled": weight_decay * lr,
            "independent": weight_decay,
            "palm": weight_decay * lr * lr,
        }.get(method)
        if shrink is None:
            raise ValueError(f"Invalid weight decay method: {method}")
        torch._foreach_add_(params, params, alpha=-shrink)
