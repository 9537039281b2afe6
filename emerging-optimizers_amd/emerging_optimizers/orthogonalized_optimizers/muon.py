"""Muon (MomentUm Orthogonalized by Newton-schulz) on top of :class:`OrthogonalizedOptimizer`.

Constructor arguments, defaults, read-only properties and the scale-factor rules follow the reference's
``Muon`` (orthogonalized_optimizers/muon.py:37-216).

A float32 parameter on a gfx950 GPU with both dims multiples of 8 is orthogonalised on the hand-written kernels
under the default matmul precision "medium", whatever ``use_syrk`` says (see ``muon_utils.newton_schulz``): the
reference's flag chooses between two library back ends for the same products, here the kernel library makes that
choice itself.  ``use_syrk=True`` keeps its checks: the reference whitelists NVIDIA SM versions at that point
(muon.py:101-115), here the condition is "a gfx950 device and a loadable libmi_ns.so", and a GPU without the
library is an error rather than a downgrade.
"""

from __future__ import annotations

import logging
from typing import Literal, Optional

import torch
from torch.optim.optimizer import ParamsT

from emerging_optimizers import hip_kernels
from emerging_optimizers.mixin import WeightDecayT
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from emerging_optimizers.orthogonalized_optimizers.muon_utils import NSCoeffT
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer, _args_doc
from emerging_optimizers.utils import FP32MatmulPrecT
from emerging_optimizers.weight_update_hooks import WeightUpdateHook
from emerging_optimizers.weight_update_hooks.base import HookStateT


__all__ = ["Muon", "get_muon_scale_factor"]

_log = logging.getLogger(__name__)

MuonScaleT = Literal["shape_scaling", "spectral", "unit_rms_norm"]

# Switch of the one-call parameter update (momentum + Nesterov + Newton-Schulz + weight update in the library,
# see hip_kernels.fused_muon_update).  Results agree with the statement-by-statement path to float32 rounding of
# the elementwise parts; set to False to run the latter.
FUSED_MUON_STEP = True


def get_muon_scale_factor(size_out: int, size_in: int, mode: MuonScaleT = "spectral") -> float:
    """Multiplier applied to the orthogonalised update of a ``(size_out, size_in)`` weight.

    * ``"shape_scaling"``: ``sqrt(max(1, size_out / size_in))`` (original Muon post)
    * ``"spectral"``: ``sqrt(max(size_out, size_in))`` (learning rates transfer from AdamW, arXiv:2502.16982)
    * ``"unit_rms_norm"``: ``sqrt(size_out / size_in)`` (Scion, arXiv:2502.07529)
    """
    if mode == "spectral":
        return max(size_out, size_in) ** 0.5
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "unit_rms_norm":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for Muon update scale factor: {mode}")


def _resolve_use_syrk(requested: bool) -> bool:
    if not requested:
        return False
    if not torch.cuda.is_available():
        _log.error("use_syrk needs a GPU; none is visible. Setting use_syrk to False.")
        return False
    if not hip_kernels.HAS_HIP_KERNELS:
        # A GPU is present and the kernels were asked for: refusing is better than a silent slow path.
        raise RuntimeError("use_syrk=True but libmi_ns.so could not be loaded; build it with `make -C csrc`.")
    arch = getattr(torch.cuda.get_device_properties(torch.cuda.current_device()), "gcnArchName", "")
    if not arch.startswith("gfx950"):
        _log.error("The HIP kernels are built for gfx950 only, found %r. Setting use_syrk to False.", arch)
        return False
    return True


class Muon(OrthogonalizedOptimizer[HookStateT]):
    """Momentum SGD whose update for every 2-D parameter is replaced by (approximately) the nearest
    semi-orthogonal matrix, computed with a few Newton-Schulz iterations, then rescaled by shape.

    Use it for hidden-layer weight matrices only; embeddings, the output head and 1-D parameters belong to
    an element-wise optimizer such as AdamW.

    Args:
        {_args_doc}
        coefficient_type: Newton-Schulz coefficient family ("simple", "quintic", "polar_express", "cans",
            "aol", "deepseekv4", "cubic5", "custom").
        num_ns_steps: number of Newton-Schulz iterations (at least 1).
        scale_mode: see :func:`get_muon_scale_factor`.
        extra_scale_factor: further multiplier of the update (0.2 roughly matches AdamW's update RMS).
        use_syrk: ask for the lower-triangle (SYRK) kernels explicitly; raises when a GPU is present but the kernel
            library is not.  The default False gives the same results on a gfx950 GPU (the library chooses its
            kernels by shape); the flag still selects the ``*_tsyrk`` step functions where steps run one by one.
        group_same_shape: one batched orthogonalisation per distinct parameter shape (see the base class).
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
        fp32_matmul_prec: FP32MatmulPrecT = "medium",
        coefficient_type: NSCoeffT = "quintic",
        num_ns_steps: int = 5,
        scale_mode: MuonScaleT = "spectral",
        extra_scale_factor: float = 1.0,
        use_syrk: bool = False,
        weight_update_hook: Optional[WeightUpdateHook[HookStateT]] = None,
        group_same_shape: bool = False,
    ) -> None:
        if num_ns_steps < 1:
            raise ValueError(f"num_ns_steps must be at least 1, got {num_ns_steps}")
        use_syrk = _resolve_use_syrk(use_syrk)
        self._num_ns_steps = num_ns_steps
        self._coefficient_type = coefficient_type
        self._scale_mode = scale_mode
        self._extra_scale_factor = extra_scale_factor
        self._use_syrk = use_syrk

        def scaled_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            _log.debug(
                "orthogonalize: %s steps, %s coefficients, scale mode %s, extra scale %s",
                num_ns_steps, coefficient_type, scale_mode, extra_scale_factor,
            )  # fmt: skip
            scale = get_muon_scale_factor(grad.size(-2), grad.size(-1), mode=scale_mode)
            ns = muon_utils.newton_schulz
            if ns is muon_utils._ORIGINAL_NEWTON_SCHULZ:
                # own driver: let the last kernel's epilogue apply both factors
                return ns(
                    grad,
                    steps=num_ns_steps,
                    coefficient_type=coefficient_type,
                    use_syrk=use_syrk,
                    _out_scale=scale * extra_scale_factor,
                )
            return ns(grad, steps=num_ns_steps, coefficient_type=coefficient_type, use_syrk=use_syrk) * scale * extra_scale_factor

        super().__init__(
            params,
            lr,
            momentum,
            nesterov=nesterov,
            weight_decay=weight_decay,
            weight_decay_method=weight_decay_method,
            fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn,
            weight_update_hook=weight_update_hook,
            group_same_shape=group_same_shape,
        )
        self._own_scaled_orthogonalize_fn = scaled_orthogonalize_fn

    def _fused_update(
        self, p: torch.Tensor, grad: torch.Tensor, buf: torch.Tensor, lr: float, beta: float, weight_decay: float
    ) -> bool:
        """Whole update of one 2-D parameter in a single library call, when nothing needs the intermediates.

        Taken for float32 parameters on a gfx950 GPU with both dims multiples of 8 under matmul precision "medium",
        with the library's own ``newton_schulz``, no subclass or weight-update hooks, and a weight decay that only
        scales the parameter (every method except ``"l2"``, which modifies the gradient).
        """
        if not (FUSED_MUON_STEP and self.fp32_matmul_prec == "medium" and p.ndim == 2 and p.is_cuda):
            return False
        if self.scaled_orthogonalize_fn is not self._own_scaled_orthogonalize_fn or not self._update_is_plain():
            return False
        if muon_utils.newton_schulz is not muon_utils._ORIGINAL_NEWTON_SCHULZ:
            return False
        if not muon_utils._fused_path_ok(grad, grad.size(-2) > grad.size(-1), None):
            return False
        tensors = (p, grad, buf)
        if not all(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.shape == p.shape for t in tensors):
            return False
        if len({t.data_ptr() for t in tensors}) != 3 or not isinstance(lr, (int, float)):
            return False
        shrink = 0.0
        if weight_decay != 0.0:
            shrink = {
                "decoupled": weight_decay * lr,
                "independent": weight_decay,
                "palm": weight_decay * lr * lr,
            }.get(self.weight_decay_method)
            if shrink is None or shrink == 1.0:
                return False  # "l2" changes the gradient; a decay of exactly 1 is left to the generic statements
        coeffs = muon_utils._schedule(self._num_ns_steps, self._coefficient_type, None)
        scale = get_muon_scale_factor(p.size(-2), p.size(-1), mode=self._scale_mode) * self._extra_scale_factor
        hip_kernels.fused_muon_update(
            p.data, grad, buf, coeffs, beta=beta, nesterov=self.nesterov, param_decay=1.0 - shrink,
            update_scale=-lr * scale,
        )  # fmt: skip
        return True


def _read_only(name: str) -> property:
    def getter(self):
        return getattr(self, "_" + name)

    def setter(self, _value):
        raise AttributeError(f"Cannot set `{name}` post-initialization.")

    return property(getter, setter)


for _name in ("num_ns_steps", "coefficient_type", "scale_mode", "extra_scale_factor", "use_syrk"):
    setattr(Muon, _name, _read_only(_name))

Muon.__doc__ = Muon.__doc__.format(_args_doc=_args_doc)  # type: ignore[union-attr]
