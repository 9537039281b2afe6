"""Muon with a second-moment normalisation between the orthogonalisation and Muon's shape scaling.

Behaviour follows the reference's ``AdaptiveMuon`` (orthogonalized_optimizers/adaptive_muon.py:38-331):

* ``"adamuon"`` (arXiv:2507.11005): element-wise EMA ``v`` of ``O**2``; update ``O / (sqrt(v) + eps)``.
* ``"normuon"`` (arXiv:2510.05491): EMA of the mean of ``O**2`` along the longer side; update
  ``O * rsqrt(max(v, eps))`` rescaled to the Frobenius norm of ``O``.
* ``"namo"`` (arXiv:2602.17080): scalar EMA ``v`` of ``||G||_F**2``; update ``O * ||M||_F / (sqrt(v) + eps)`` with
  ``M`` the matrix handed to Newton-Schulz.

``O`` is the raw Newton-Schulz output; Muon's scale factor multiplies the normalised update afterwards.
``use_syrk`` is an addition (the reference fixes False); it is handed to ``newton_schulz``, which under matmul
precision "medium" runs float32 matrices on a gfx950 GPU on the kernels for either value.
"""

from __future__ import annotations

import logging
from typing import Callable, Literal, Optional

import torch
from torch.optim.optimizer import ParamsT

from emerging_optimizers import utils
from emerging_optimizers.mixin import WeightDecayT
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from emerging_optimizers.orthogonalized_optimizers.muon import MuonScaleT, _resolve_use_syrk, get_muon_scale_factor
from emerging_optimizers.orthogonalized_optimizers.muon_utils import NSCoeffT
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer
from emerging_optimizers.utils import FP32MatmulPrecT


__all__ = ["AdaptiveMuon", "Moment2MethodT"]

Moment2MethodT = Literal["adamuon", "normuon", "namo"]

_log = logging.getLogger(__name__)


def _long_side(shape: torch.Size) -> int:
    """The dimension NorMuon averages over: the last one unless the matrix is wider than tall."""
    return -1 if shape[-2] >= shape[-1] else -2


class AdaptiveMuon(OrthogonalizedOptimizer):
    """Args are those of :class:`Muon` (all required positionally up to ``weight_decay``), plus:

    Args:
        moment2_method: "adamuon", "normuon" or "namo" (see the module docstring)
        beta2: EMA coefficient of the second moment
        eps: stabiliser of the division
        use_syrk: forwarded to ``newton_schulz``
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float,
        momentum: float,
        weight_decay: float,
        *,
        nesterov: bool = False,
        weight_decay_method: WeightDecayT = "decoupled",
        fp32_matmul_prec: FP32MatmulPrecT = "medium",
        coefficient_type: NSCoeffT = "quintic",
        num_ns_steps: int = 5,
        scale_mode: MuonScaleT = "spectral",
        extra_scale_factor: float = 1.0,
        moment2_method: Moment2MethodT = "adamuon",
        beta2: float = 0.95,
        eps: float = 1e-8,
        use_syrk: bool = False,
    ) -> None:
        if moment2_method == "namo" and weight_decay_method == "l2":
            raise ValueError('moment2_method="namo" is incompatible with weight_decay_method="l2"')
        if num_ns_steps < 1:
            raise ValueError(f"num_ns_steps must be at least 1, got {num_ns_steps}")
        use_syrk = _resolve_use_syrk(use_syrk)
        self.scale_mode = scale_mode
        self.extra_scale_factor = extra_scale_factor
        self.moment2_method = moment2_method

        def raw_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            return muon_utils.newton_schulz(
                grad, steps=num_ns_steps, coefficient_type=coefficient_type, use_syrk=use_syrk
            )

        super().__init__(
            params,
            lr,
            momentum,
            weight_decay,
            nesterov=nesterov,
            weight_decay_method=weight_decay_method,
            fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=raw_orthogonalize_fn,
        )
        for group in self.param_groups:
            group.setdefault("beta2", beta2)
            group.setdefault("eps", eps)

    @torch.no_grad()
    def _init_group(self, group: dict, skip_non_grad_params: bool = True) -> None:
        for p in group["params"]:
            if (skip_non_grad_params and p.grad is None) or len(self.state[p]) != 0:
                continue
            state = self.state[p]
            state["momentum_buffer"] = torch.zeros_like(p.data)
            if self.moment2_method == "adamuon":
                state["moment2_buffer"] = torch.zeros_like(p.data)
            elif self.moment2_method == "normuon":
                if p.data.ndim != 2:
                    raise ValueError(
                        f"{self.__class__.__name__} only supports 2D parameters, got shape {tuple(p.data.shape)}"
                    )
                shape = list(p.data.shape)
                shape[_long_side(p.data.shape)] = 1
                state["moment2_buffer"] = torch.zeros(shape, dtype=p.data.dtype, device=p.data.device)
            elif self.moment2_method == "namo":
                state["moment2_buffer"] = torch.zeros(1, dtype=p.data.dtype, device=p.data.device)
            else:
                raise TypeError(f"Invalid second moment method: {self.moment2_method}")

    def _apply_muon_scale(self, update: torch.Tensor, size_out: int, size_in: int) -> torch.Tensor:
        return update * get_muon_scale_factor(size_out, size_in, mode=self.scale_mode) * self.extra_scale_factor

    def _apply_moment2_normalization(
        self,
        orth_grad: torch.Tensor,
        moment2: torch.Tensor,
        beta2: float,
        eps: float,
        *,
        raw_grad: Optional[torch.Tensor] = None,
        pre_orth_grad: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """Update ``moment2`` in place and return the normalised (not yet Muon-scaled) update."""
        if self.moment2_method == "adamuon":
            moment2.lerp_(orth_grad.square(), 1 - beta2)
            return orth_grad / (moment2.sqrt() + eps)
        if self.moment2_method == "normuon":
            moment2.lerp_(orth_grad.square().mean(dim=_long_side(orth_grad.shape), keepdim=True), 1 - beta2)
            update = orth_grad * moment2.clamp_min(eps).rsqrt_()
            keep = torch.linalg.vector_norm(orth_grad) / torch.linalg.vector_norm(update).clamp_min(eps)
            return update * keep
        if self.moment2_method == "namo":
            if raw_grad is None or pre_orth_grad is None:
                raise RuntimeError("NAMO requires raw_grad and pre_orth_grad")
            moment2.lerp_(torch.linalg.vector_norm(raw_grad).square(), 1 - beta2)
            return orth_grad * (torch.linalg.vector_norm(pre_orth_grad) / (moment2.sqrt() + eps))
        raise TypeError(f"Invalid second moment method: {self.moment2_method}")

    @torch.no_grad()
    def step(self, closure: Optional[Callable[[], float]] = None) -> Optional[float]:
        if closure is not None:
            raise ValueError("closure is not supported")
        namo = self.moment2_method == "namo"
        for group in self.param_groups:
            self._init_group(group)
            for p in group["params"]:
                if p.dim() != 2:
                    raise ValueError(f"{self.__class__.__name__} only supports 2D parameters")
                grad = p.grad
                if grad is None:
                    continue
                state = self.state[p]
                buf = state["momentum_buffer"]
                self._apply_weight_decay_inplace(p, grad, group["lr"], group["weight_decay"])
                raw_grad = grad if namo else None
                buf.lerp_(grad, 1 - group["momentum"])
                direction = grad.lerp(buf, group["momentum"]) if self.nesterov else buf
                with utils.fp32_matmul_precision(self.fp32_matmul_prec):
                    orth = self.orthogonalize(p, direction, **{k: v for k, v in group.items() if k != "params"})
                update = self._apply_moment2_normalization(
                    orth,
                    state["moment2_buffer"],
                    group["beta2"],
                    group["eps"],
                    raw_grad=raw_grad,
                    pre_orth_grad=direction if namo else None,
                )
                update = self._apply_muon_scale(update, update.size(-2), update.size(-1))
                self.pre_weight_update_fn_inplace(p, update)
                p.add_(update, alpha=-group["lr"])
                self.post_weight_update_fn_inplace(p)
        return None
