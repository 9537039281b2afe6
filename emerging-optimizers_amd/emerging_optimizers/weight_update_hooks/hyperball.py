"""Keep a weight on a sphere of fixed Frobenius norm across the update (reference: weight_update_hooks/hyperball.py:24-63)."""

from __future__ import annotations

import math

import torch


__all__ = ["HyperballHook"]


class HyperballHook:
    """Before the update: rescale the update to ``radius``.  After it: rescale the weight to ``radius``.

    A tensor whose norm is below ``eps`` has no direction to keep and is set to exactly zero.
    """

    def __init__(self, radius: float, eps: float = 1e-15) -> None:
        if not (math.isfinite(eps) and eps > 0.0):
            raise ValueError(f"eps must be finite and positive, got {eps}")
        if not (math.isfinite(radius) and radius >= eps):
            raise ValueError(f"radius must be finite and at least eps={eps}, got {radius}")
        self.radius = radius
        self.eps = eps

    def _to_radius_(self, t: torch.Tensor) -> None:
        norm = torch.linalg.vector_norm(t, dtype=torch.float32)
        factor = self.radius / norm.clamp_min(self.eps)
        factor = torch.where(norm < self.eps, torch.zeros_like(factor), factor)
        t.mul_(factor.to(t.dtype))

    def pre_weight_update_inplace(self, p: torch.Tensor, update: torch.Tensor) -> None:
        self._to_radius_(update)
        return None

    def post_weight_update_inplace(self, p: torch.Tensor, pre_update_state: None) -> None:
        self._to_radius_(p)
