"""PolarGrad: the orthogonalised momentum scaled by (an estimate of) its nuclear norm (arXiv:2505.21799).

Behaviour follows the reference's ``PolarGrad`` class (orthogonalized_optimizers/polargrad.py:33-118): the update
is ``msign(G) * <msign(G), G> * extra_scale_factor``; the inner product equals the nuclear norm of ``G`` when the
orthogonalisation is exact.  Default matmul precision is "highest", as in the reference; ``num_ns_steps = 0`` is
allowed (the update is then ``G/||G|| * <G/||G||, G>``).  ``use_syrk`` is an addition, handed to ``newton_schulz``
(the kernels run under "medium" only).
The eigendecomposition-based one-sided variants of that file are not part of this package.
"""

from __future__ import annotations

import torch
from torch.optim.optimizer import ParamsT

from emerging_optimizers.mixin import WeightDecayT
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from emerging_optimizers.orthogonalized_optimizers.muon import _resolve_use_syrk
from emerging_optimizers.orthogonalized_optimizers.muon_utils import NSCoeffT
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer, _args_doc
from emerging_optimizers.utils import FP32MatmulPrecT


__all__ = ["PolarGrad"]


class PolarGrad(OrthogonalizedOptimizer):
    """Steepest descent in the spectral norm with the nuclear-norm step length, decoupled weight decay by default.

    Args:
        {_args_doc}
        coefficient_type: Newton-Schulz coefficient family
        num_ns_steps: Newton-Schulz iterations (0 skips the iteration, for exact-match tests)
        extra_scale_factor: extra multiplier of the update (0.2 roughly matches AdamW's update RMS, arXiv:2502.16982)
        use_syrk: forwarded to ``newton_schulz`` (not in the reference)
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float = 3e-4,
        momentum: float = 0.95,
        weight_decay: float = 0.01,
        *,
        nesterov: bool = False,
        weight_decay_method: WeightDecayT = "decoupled",
        fp32_matmul_prec: FP32MatmulPrecT = "highest",
        coefficient_type: NSCoeffT = "quintic",
        num_ns_steps: int = 5,
        extra_scale_factor: float = 1.0,
        use_syrk: bool = False,
    ) -> None:
        if num_ns_steps < 0:
            raise ValueError(f"num_ns_steps must be positive, got {num_ns_steps}")
        use_syrk = _resolve_use_syrk(use_syrk)

        def scaled_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            orth = muon_utils.newton_schulz(grad, steps=num_ns_steps, coefficient_type=coefficient_type, use_syrk=use_syrk)
            return orth * (orth * grad).sum() * extra_scale_factor

        super().__init__(
            params,
            lr,
            momentum,
            nesterov=nesterov,
            weight_decay=weight_decay,
            weight_decay_method=weight_decay_method,
            fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn,
        )


PolarGrad.__doc__ = PolarGrad.__doc__.format(_args_doc=_args_doc)  # type: ignore[union-attr]
