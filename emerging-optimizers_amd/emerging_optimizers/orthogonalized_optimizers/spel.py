"""SPEL: spectral steepest descent on the Stiefel manifold (arXiv:2601.21487).

Behaviour follows the reference's ``Spel`` (orthogonalized_optimizers/spel.py:31-129): the momentum is
orthogonalised without any scale factor, the weight takes the usual step, and the updated weight is itself
re-orthogonalised in place, ``x <- msign((1 - lr wd) x - lr msign(momentum))``.  Two Newton-Schulz calls per
parameter and step.  ``use_syrk`` is an addition (the reference fixes False); it is handed to ``newton_schulz``, which under matmul
precision "medium" runs float32 matrices on a gfx950 GPU on the kernels for either value.
"""

from __future__ import annotations

import torch
from torch.optim.optimizer import ParamsT

from emerging_optimizers import utils
from emerging_optimizers.mixin import WeightDecayT
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from emerging_optimizers.orthogonalized_optimizers.muon import _resolve_use_syrk
from emerging_optimizers.orthogonalized_optimizers.muon_utils import NSCoeffT
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer, _args_doc
from emerging_optimizers.utils import FP32MatmulPrecT


__all__ = ["Spel"]


class Spel(OrthogonalizedOptimizer):
    """Momentum SGD with an orthogonalised step and a re-orthogonalised weight (parameters stay near orthogonal).

    Weight decay still matters: it sets the mixing ratio of old weight and step before the outer projection.

    Args:
        {_args_doc}
        coefficient_type: Newton-Schulz coefficient family, used for both projections
        num_ns_steps: Newton-Schulz iterations of each projection (at least 1)
        use_syrk: forwarded to both ``newton_schulz`` calls (not in the reference, which fixes False)
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float = 3e-4,
        momentum: float = 0.95,
        weight_decay: float = 0.1,
        *,
        nesterov: bool = False,
        weight_decay_method: WeightDecayT = "decoupled",
        fp32_matmul_prec: FP32MatmulPrecT = "medium",
        coefficient_type: NSCoeffT = "quintic",
        num_ns_steps: int = 5,
        use_syrk: bool = False,
    ) -> None:
        if num_ns_steps < 1:
            raise ValueError(f"num_ns_steps must be at least 1, got {num_ns_steps}")
        use_syrk = _resolve_use_syrk(use_syrk)

        def scaled_orthogonalize_fn(x: torch.Tensor) -> torch.Tensor:
            return muon_utils.newton_schulz(x, steps=num_ns_steps, coefficient_type=coefficient_type, use_syrk=use_syrk)

        super().__init__(
            params,
            lr,
            momentum,
            weight_decay,
            nesterov=nesterov,
            weight_decay_method=weight_decay_method,
            fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn,
        )

    def post_weight_update_fn_inplace(self, p: torch.Tensor) -> None:
        """Outer projection: replace the freshly updated weight by its orthogonal polar factor."""
        with utils.fp32_matmul_precision(self.fp32_matmul_prec):
            p.copy_(self.scaled_orthogonalize_fn(p))


Spel.__doc__ = Spel.__doc__.format(_args_doc=_args_doc)  # type: ignore[union-attr]
