"""Momentum-SGD skeleton whose update is passed through an orthogonalisation function.

Behaviour follows the reference's ``OrthogonalizedOptimizer``
(orthogonalized_optimizers/orthogonalized_optimizer.py:47-272): per parameter, in this order,
weight decay -> EMA momentum -> optional Nesterov blend -> ``orthogonalize`` (under the configured float32
matmul precision) -> pre hooks -> ``p += -lr * update`` -> post hooks.  The only optimizer state is
``momentum_buffer``.
"""

from __future__ import annotations

import logging
from typing import Any, Callable, Generic, Optional

import torch
from torch.optim.optimizer import Optimizer, ParamsT

from emerging_optimizers import utils
from emerging_optimizers.mixin import WeightDecayMixin, WeightDecayT
from emerging_optimizers.utils import FP32MatmulPrecT
from emerging_optimizers.weight_update_hooks import NoOpWeightUpdateHook, WeightUpdateHook
from emerging_optimizers.weight_update_hooks.base import HookStateT


_log = logging.getLogger(__name__)

_args_doc = """params: parameters (or parameter-group dicts) to optimize
        lr: learning rate of the inner SGD
        momentum: EMA coefficient of the momentum buffer (``buf = momentum * buf + (1 - momentum) * grad``)
        weight_decay: weight-decay strength; how it is applied is set by ``weight_decay_method``
        nesterov: blend the fresh gradient with the buffer once more before orthogonalising
        weight_decay_method: one of the flavours of :class:`~emerging_optimizers.mixin.WeightDecayMixin`
        fp32_matmul_prec: float32 matmul precision in force while orthogonalising ("medium" = bf16 kernels)
        weight_update_hook: optional object called right before and after the in-place weight update
"""


class OrthogonalizedOptimizer(WeightDecayMixin, Optimizer, Generic[HookStateT]):
    """SGD-with-momentum whose per-parameter update goes through ``scaled_orthogonalize_fn`` first.

    Subclasses usually only supply ``scaled_orthogonalize_fn``.  To treat fused parameters (e.g. a stacked
    QKV weight) piecewise, override :meth:`orthogonalize`, split ``grad`` there and call
    ``self.scaled_orthogonalize_fn`` on each piece (it also accepts a stacked 3-D tensor).

    Args:
        {_args_doc}
        scaled_orthogonalize_fn: maps the momentum tensor to the update; identity when omitted.
        group_same_shape: orthogonalise all 2-D parameters of one shape (within a parameter group) in one
            batched call instead of one call each.  Not in the reference, whose loop
            (orthogonalized_optimizer.py:175-210) is serial; pays for many small matrices (attention heads kept
            as separate parameters), where single calls are bound by launch latency.
        **kwargs: extra per-group defaults, stored unchecked.
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float,
        momentum: float,
        weight_decay: float,
        *,
        nesterov: bool,
        weight_decay_method: WeightDecayT,
        fp32_matmul_prec: FP32MatmulPrecT,
        scaled_orthogonalize_fn: Optional[Callable] = None,
        weight_update_hook: Optional[WeightUpdateHook[HookStateT]] = None,
        group_same_shape: bool = False,
        **kwargs: Any,
    ):
        self._group_same_shape = bool(group_same_shape)
        if scaled_orthogonalize_fn is None:
            _log.warning("scaled_orthogonalize_fn not provided. Using noop")
            scaled_orthogonalize_fn = torch.nn.Identity()
        self.fp32_matmul_prec = fp32_matmul_prec
        self.nesterov = nesterov
        self.weight_decay_method = weight_decay_method
        self._weight_update_hook = weight_update_hook if weight_update_hook is not None else NoOpWeightUpdateHook()
        super().__init__(params, dict(lr=lr, momentum=momentum, weight_decay=weight_decay, **kwargs))
        self.scaled_orthogonalize_fn = scaled_orthogonalize_fn

    @torch.no_grad()
    def _init_group(self, group: dict, skip_non_grad_params: bool = True) -> None:
        """Create the zero momentum buffer of every parameter of ``group`` that does not have one yet."""
        for p in group["params"]:
            if p.grad is None and skip_non_grad_params:
                continue
            state = self.state[p]
            if not state:
                state["momentum_buffer"] = torch.zeros_like(p.data)

    @torch.no_grad()
    def step(self, closure: Optional[Callable[[], float]] = None) -> Optional[float]:
        """One optimisation step.  ``closure`` is not supported and must be ``None``."""
        if closure is not None:
            raise ValueError("closure is not supported")
        for group in self.param_groups:
            self._init_group(group)
            lr, beta = group["lr"], group["momentum"]
            extras = {k: v for k, v in group.items() if k != "params"}
            shared = self._shapes_to_batch(group)
            batches: dict = {}
            for p in group["params"]:
                grad = p.grad
                if grad is None:
                    continue
                buf = self.state[p]["momentum_buffer"]
                key = (tuple(p.shape), p.dtype, p.device)
                if key not in shared and self._fused_update(p, grad, buf, lr, beta, group["weight_decay"]):
                    continue
                if key in shared:
                    batches.setdefault(key, []).append(p)
                    continue
                self._apply_weight_decay_inplace(p, grad, lr, group["weight_decay"])
                buf.lerp_(grad, 1 - beta)
                direction = grad.lerp(buf, beta) if self.nesterov else buf
                with utils.fp32_matmul_precision(self.fp32_matmul_prec):
                    update = self.orthogonalize(p, direction, **extras)
                self._apply_update(p, update, lr)
            for members in batches.values():
                # Same statements as above, as multi-tensor launches, around one batched orthogonalisation in
                # which every matrix of the stack is treated exactly as it would be alone.
                grads = [p.grad for p in members]
                bufs = [self.state[p]["momentum_buffer"] for p in members]
                self._apply_weight_decay_foreach_inplace(members, grads, lr, group["weight_decay"])
                torch._foreach_lerp_(bufs, grads, 1 - beta)
                directions = torch._foreach_lerp(grads, bufs, beta) if self.nesterov else bufs
                with utils.fp32_matmul_precision(self.fp32_matmul_prec):
                    updates = self.scaled_orthogonalize_fn(torch.stack(list(directions)))
                if self._update_is_plain():
                    torch._foreach_add_(members, list(updates.unbind(0)), alpha=-lr)
                else:
                    for p, update in zip(members, updates):
                        self._apply_update(p, update, lr)
        return None

    def _apply_update(self, p: torch.Tensor, update: torch.Tensor, lr: float) -> None:
        self.pre_weight_update_fn_inplace(p, update)
        hook_state = self._weight_update_hook.pre_weight_update_inplace(p, update)
        p.add_(update, alpha=-lr)
        self.post_weight_update_fn_inplace(p)
        self._weight_update_hook.post_weight_update_inplace(p, hook_state)

    def _shapes_to_batch(self, group: dict) -> set:
        """(shape, dtype, device) keys shared by two or more 2-D parameters with gradients, when batching is on
        and ``orthogonalize`` is the base implementation (an override may treat a parameter piecewise)."""
        if not self._group_same_shape or type(self).orthogonalize is not OrthogonalizedOptimizer.orthogonalize:
            return set()
        seen: dict = {}
        for p in group["params"]:
            if p.grad is not None and p.dim() == 2:
                key = (tuple(p.shape), p.dtype, p.device)
                seen[key] = seen.get(key, 0) + 1
        return {k for k, n in seen.items() if n > 1}

    def _fused_update(
        self, p: torch.Tensor, grad: torch.Tensor, buf: torch.Tensor, lr: float, beta: float, weight_decay: float
    ) -> bool:
        """Hook for subclasses that can do the whole update of ``p`` in one library call.

        Return ``True`` after having updated ``buf`` and ``p`` exactly as the statements of :meth:`step` that
        follow would have; return ``False`` (the default) to let :meth:`step` run them.
        """
        return False

    def _update_is_plain(self) -> bool:
        """No subclass or hook needs to see the update tensor, so it does not have to exist in memory."""
        cls = type(self)
        return (
            cls.orthogonalize is OrthogonalizedOptimizer.orthogonalize
            and cls.pre_weight_update_fn_inplace is OrthogonalizedOptimizer.pre_weight_update_fn_inplace
            and cls.post_weight_update_fn_inplace is OrthogonalizedOptimizer.post_weight_update_fn_inplace
            and type(self._weight_update_hook) is NoOpWeightUpdateHook
        )

    def orthogonalize(self, p: torch.Tensor, grad: torch.Tensor, **kwargs: Any) -> torch.Tensor:
        """Turn the momentum ``grad`` of parameter ``p`` into the update.

        The base version accepts 2-D tensors only and applies ``scaled_orthogonalize_fn``.  ``p`` and the
        parameter-group entries in ``kwargs`` are there for overrides that need per-parameter attributes
        (fused QKV splits, reshaped convolution weights, per-head stacking).
        """
        if grad.ndim != 2:
            raise ValueError("Only 2D parameters are supported.")
        return self.scaled_orthogonalize_fn(grad)

    def pre_weight_update_fn_inplace(self, p: torch.Tensor, update: torch.Tensor) -> None:
        """Subclass hook, called with the final update just before ``p.add_(update, alpha=-lr)``."""

    def post_weight_update_fn_inplace(self, p: torch.Tensor) -> None:
        """Subclass hook, called with the already updated parameter."""


OrthogonalizedOptimizer.__doc__ = OrthogonalizedOptimizer.__doc__.format(_args_doc=_args_doc)  # type: ignore[union-attr]
