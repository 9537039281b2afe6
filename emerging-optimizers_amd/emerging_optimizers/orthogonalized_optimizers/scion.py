"""Scion: momentum SGD whose step is the spectral-norm LMO, i.e. a scaled orthogonalised momentum.

Constructor arguments and behaviour follow the reference's ``Scion``
(orthogonalized_optimizers/scion.py:31-106): no Nesterov blend, and the Frank-Wolfe step is obtained from the
base class by fixing decoupled weight decay at 1, so each step is
``p <- (1 - lr) p - lr * spectral_radius * sqrt(out / in) * msign(momentum)``.
``use_syrk`` is an addition (the reference fixes False); it is handed to ``newton_schulz``, which under matmul
precision "medium" runs float32 matrices on a gfx950 GPU on the kernels for either value.
"""

from __future__ import annotations

import logging

import torch
from torch.optim.optimizer import ParamsT

from emerging_optimizers.orthogonalized_optimizers import muon_utils
from emerging_optimizers.orthogonalized_optimizers.muon import _resolve_use_syrk, get_muon_scale_factor
from emerging_optimizers.orthogonalized_optimizers.muon_utils import NSCoeffT
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer
from emerging_optimizers.utils import FP32MatmulPrecT


__all__ = ["Scion"]

_log = logging.getLogger(__name__)


class Scion(OrthogonalizedOptimizer):
    """Stochastic conditional descent with operator norms (arXiv:2502.07529) for 2-D hidden-layer weights.

    Args:
        params: parameters (or parameter-group dicts) to optimize; all must be 2-D
        lr: step size of the Frank-Wolfe step
        momentum: EMA coefficient of the momentum buffer
        fp32_matmul_prec: float32 matmul precision in force while orthogonalising ("medium" = bf16 kernels)
        coefficient_type: Newton-Schulz coefficient family
        num_ns_steps: Newton-Schulz iterations (at least 1)
        spectral_radius: radius of the spectral-norm ball the LMO is scaled to
        use_syrk: forwarded to ``newton_schulz`` (not in the reference, which fixes False)
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float = 3e-4,
        momentum: float = 0.95,
        *,
        fp32_matmul_prec: FP32MatmulPrecT = "medium",
        coefficient_type: NSCoeffT = "quintic",
        num_ns_steps: int = 5,
        spectral_radius: float = 1.0,
        use_syrk: bool = False,
    ) -> None:
        if num_ns_steps < 1:
            raise ValueError(f"num_ns_steps must be at least 1, got {num_ns_steps}")
        use_syrk = _resolve_use_syrk(use_syrk)
        _log.info("Scion fixes weight_decay=1 (decoupled) and nesterov=False: the step is a Frank-Wolfe step.")

        def scaled_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            width = get_muon_scale_factor(grad.size(-2), grad.size(-1), mode="unit_rms_norm")
            ns = muon_utils.newton_schulz
            kwargs = dict(steps=num_ns_steps, coefficient_type=coefficient_type, use_syrk=use_syrk)
            if ns is muon_utils._ORIGINAL_NEWTON_SCHULZ:
                return ns(grad, _out_scale=width * spectral_radius, **kwargs)  # scale folded into the last kernel
            return ns(grad, **kwargs) * width * spectral_radius

        super().__init__(
            params,
            lr,
            momentum,
            1,
            nesterov=False,
            weight_decay_method="decoupled",
            fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn,
        )
