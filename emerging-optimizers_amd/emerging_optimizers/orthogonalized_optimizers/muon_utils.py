"""Newton-Schulz orthogonalisation: host driver over the gfx950 kernels.

Public surface and behaviour follow ``emerging_optimizers/orthogonalized_optimizers/muon_utils.py`` of the
reference (function names, arguments, exception types/messages, the late-bound step functions), so callers
and tests written against it run unchanged.  What differs is where the work goes:

* float32 GPU input, matmul precision ``"medium"``, both dims multiples of 8 -> one call into
  ``libmi_ns.so`` (normalise, bf16 cast, all steps, float32 result) -- the hot path.  ``use_syrk`` does not
  select it: in the reference that flag only picks between two library back ends for the same products
  (its default ``False`` means cuBLAS GEMMs); here the library itself decides which of its kernels forms
  a product, so both values of the flag give the same, bit-identical, result on such input.
* the four step functions on bf16 GPU operands with both dims multiples of 8 -> HIP lower-triangle product +
  HIP GEMM/AXPY kernels, one launch per product, with the reference's rounding points (every product
  accumulated in float32 and rounded to bf16 once).
* everything else (CPU tensors, float32 arithmetic under "highest"/"high", shapes that are not multiples
  of 8) -> the same torch operators the reference uses; these are not accelerated and not part of the
  hot path.

GPU tensors never fall back silently: where the kernels apply and ``libmi_ns.so`` is missing, the call
raises.
"""

from __future__ import annotations

import logging
from typing import Any, Iterator, Literal, Sequence

import torch

from emerging_optimizers import hip_kernels, triton_kernels


__all__ = ["newton_schulz", "newton_schulz_tp", "NSCoeffT", "get_coefficient_iterator", "CoeffIterMode"]

_log = logging.getLogger(__name__)

CoeffIterMode = Literal["cycle", "repeat_last"]
NSCoeffT = Literal["simple", "quintic", "polar_express", "cans", "aol", "deepseekv4", "custom", "cubic5"]
Coeff = tuple[float, float, float]

# (a, b, c) per step of X <- a X + (b A + c A^2) X, A = X X^T.  Values as published by each source
# (reference table: muon_utils.py:26-90).
_SIMPLE: Coeff = (3.4445, -4.7750, 2.0315)
_COEFFICIENT_SETS: dict[str, list[Coeff]] = {
    "simple": [_SIMPLE],
    # leloykun.github.io/ponder/muon-opt-coeffs, as used by modded-nanogpt
    "quintic": [
        (4.0848, -6.8946, 2.9270),
        (3.9505, -6.3029, 2.6377),
        (3.7418, -5.5913, 2.3037),
        (2.8769, -3.1427, 1.2046),
        (2.8366, -3.0525, 1.2012),
    ],
    # Polar Express (arXiv:2505.16932), including its 1.01^degree safety division
    "polar_express": [
        (8.2051, -22.9019, 16.4607),
        (4.0664, -2.8612, 0.5184),
        (3.9096, -2.8234, 0.5250),
        (3.2856, -2.4153, 0.4853),
        (2.2779, -1.6198, 0.3985),
        (1.8726, -1.2307, 0.3585),
        (1.8564, -1.2132, 0.3568),
        (1.8750, -1.2500, 0.3750),
    ],
    # CANS (arXiv:2506.10935)
    "cans": [
        (8.4703, -25.1081, 18.6293),
        (4.1828, -3.1087, 0.5806),
        (3.9619, -2.9541, 0.5630),
        (3.2866, -2.4647, 0.5074),
        (2.2737, -1.6447, 0.4162),
    ],
    # flash-newton-schulz "AOL" set
    "aol": [
        (4.0098, -7.0585, 2.4635),
        (3.4585, -5.5479, 2.5959),
        (2.7573, -3.2939, 1.4254),
        (2.7215, -3.0494, 1.3169),
    ],
    # DeepSeek-V4: eight "simple" steps, then two (2, -1.5, 0.5)
    "deepseekv4": [_SIMPLE] * 8 + [(2.0, -1.5, 0.5)] * 2,
    # relaxed cubic schedule (arXiv:2606.00371): c == 0 selects the cubic step, no A^2 product
    "cubic5": [
        (3.3656576, -3.3420992, 0.0),
        (2.5744352, -1.4957376, 0.0),
        (2.5368962, -1.4312570, 0.0),
        (2.4418906, -1.2764040, 0.0),
        (2.2230472, -0.9630650, 0.0),
    ],
}
# Families whose schedule ends in a fixed point keep re-using their last tuple; the others wrap around.
_REPEAT_LAST = frozenset({"polar_express", "cans", "deepseekv4"})

_log_counts: dict[str, int] = {}


def _log_first_n(level: int, key: str, limit: int, msg: str, *args: Any) -> None:
    seen = _log_counts.get(key, 0)
    if seen < limit:
        _log_counts[key] = seen + 1
        _log.log(level, msg, *args)


def get_coefficient_iterator(
    steps: int,
    coefficient_sets: Sequence[Coeff],
    mode: CoeffIterMode = "cycle",
) -> Iterator[Coeff]:
    """Yield ``steps`` coefficient tuples: ``sets[i % len]`` ("cycle") or ``sets[min(i, len - 1)]`` ("repeat_last").

    Raises ``ValueError`` for an empty table or an unknown mode (both checked eagerly, as in the reference,
    muon_utils.py:93-129).
    """
    _log.debug("coefficient iterator: %s steps, mode %s, sets %s", steps, mode, coefficient_sets)
    if not coefficient_sets:
        raise ValueError("coefficient_sets must be non-empty.")
    if mode not in ("cycle", "repeat_last"):
        raise ValueError(f"Invalid mode: {mode}. Expected 'cycle' or 'repeat_last'.")
    count = len(coefficient_sets)
    if mode == "cycle":
        return (coefficient_sets[i % count] for i in range(steps))
    return (coefficient_sets[min(i, count - 1)] for i in range(steps))


def _schedule(steps: int, coefficient_type: str, custom: Sequence[Coeff] | None) -> list[Coeff]:
    table = _COEFFICIENT_SETS.get(coefficient_type)
    if table is None:
        if coefficient_type != "custom":
            raise ValueError(f"Invalid coefficient type: {coefficient_type}")
        if custom is None:
            raise ValueError("custom_coefficient_sets must be provided when coefficient_type is 'custom'.")
        table = custom
    if coefficient_type == "cubic5" and steps != len(table):
        raise ValueError(
            f"cubic5 is a fixed {len(table)}-step schedule; got steps={steps}. "
            "Use steps=5, or pass explicit custom coefficients."
        )
    mode: CoeffIterMode = "repeat_last" if coefficient_type in _REPEAT_LAST else "cycle"
    return list(get_coefficient_iterator(steps, table, mode=mode))


def distributed_normalize_p2(
    x: torch.Tensor, eps: float, group: "torch.distributed.ProcessGroup", normalize_in_double: bool = False
) -> torch.Tensor:
    """Frobenius-normalise a tensor whose shards live on the ranks of ``group`` (muon_utils.py:132-146)."""
    sq = x.double() if normalize_in_double else x
    total = (sq * sq).sum()
    torch.distributed.all_reduce(total, op=torch.distributed.ReduceOp.SUM, group=group)
    norm = total.sqrt().to(x.dtype)
    if not normalize_in_double:
        norm.clamp_min_(eps)
    return x / norm


def _normalize(x: torch.Tensor, eps: float, in_double: bool) -> torch.Tensor:
    if in_double:
        # No eps here on purpose: a norm that is zero in float64 means an all-zero input.
        norm = torch.linalg.vector_norm(x, dim=(-2, -1), keepdim=True, dtype=torch.float64)
        return x / norm.to(x.dtype)
    return torch.nn.functional.normalize(x, p=2, dim=(-2, -1), eps=eps)


def _fused_path_ok(x: torch.Tensor, transpose: bool, tp_group: Any) -> bool:
    """The single-call kernel path applies when nothing asks for per-step Python control.

    Raises ``RuntimeError`` when the input qualifies but ``libmi_ns.so`` cannot be loaded."""
    if tp_group is not None or not hip_kernels.fused_supported(x):
        return False
    if transpose != (x.size(-2) > x.size(-1)):
        return False  # caller forced the long orientation; only the step functions support that
    g = globals()
    return all(g[name] is fn for name, fn in _ORIGINAL_STEP_FNS.items())


def newton_schulz(
    x: torch.Tensor,
    steps: int,
    coefficient_type: NSCoeffT = "quintic",
    custom_coefficient_sets: list[Coeff] | None = None,
    eps: float = 1e-15,
    transpose: bool | None = None,
    tp_group: "torch.distributed.ProcessGroup | None" = None,
    use_syrk: bool = False,
    normalize_in_double: bool = False,
    *,
    _out_scale: float = 1.0,
) -> torch.Tensor:
    """Approximate the orthogonal polar factor of ``x`` with ``steps`` Newton-Schulz iterations.

    ``x`` is float32, ``(M, N)`` or batched ``(B, M, N)``.  It is Frobenius-normalised (so its spectral norm
    is at most 1) and then iterated as ``X <- a X + (b A + c A^2) X`` with ``A = X X^T`` on the orientation
    with fewer rows.  The coefficient families push singular values towards 1 quickly rather than exactly,
    so the result is ``U S' V^T`` with ``S'`` close to the identity.

    Args mirror the reference (muon_utils.py:149-274): ``coefficient_type`` one of ``NSCoeffT`` (``"custom"``
    needs ``custom_coefficient_sets``; ``"cubic5"`` needs ``steps == 5``), ``eps`` guards the float32 norm,
    ``transpose`` overrides the orientation choice, ``tp_group`` marks ``x`` as sharded along the long
    dimension, ``use_syrk`` selects the ``*_tsyrk`` step functions where the steps run one by one (effective
    only under matmul precision ``"medium"`` and for dims that are multiples of 8), ``normalize_in_double``
    reduces the norm in float64 so tiny inputs do not underflow.  ``_out_scale`` (private) is folded into the
    last kernel's epilogue.

    GPU input under ``"medium"`` with both dims multiples of 8 is orthogonalised by one library call whatever
    ``use_syrk`` says: normalisation in one pass, steps on the diagonal-shifted rounding schedule (the stored
    Gram matrix is ``A - (tr A / m) I``, so the bf16 rounding of its diagonal does not dominate the error),
    consecutive steps of wide matrices on one shared Gram matrix, float32 result without a last bf16 rounding.
    That schedule sits 3e-3 .. 7e-3 (relative Frobenius) from float32 Newton-Schulz where the reference's
    bf16 schedule -- which the step functions keep -- sits around 1e-2.

    Returns a new float32 tensor shaped like ``x``.
    """
    if x.ndim not in (2, 3):
        raise TypeError(f"Input tensor x must be 2d or 3d (batched 2d), got {x.ndim}d")
    if x.dtype != torch.float32:
        raise TypeError(f"Input tensor x must be in float32, got {x.dtype}")
    if transpose is None:
        transpose = x.size(-2) > x.size(-1)

    medium = torch.get_float32_matmul_precision() == "medium"
    if medium and x.is_cuda and _fused_path_ok(x, transpose, tp_group):
        coeffs = _schedule(steps, coefficient_type, custom_coefficient_sets)
        _log_first_n(logging.INFO, "bf16", 1, "Using BF16 I/O kernels for Newton-Schulz iteration.")
        return hip_kernels.fused_newton_schulz(x, coeffs, eps, normalize_in_double, _out_scale)

    work = x.mT if transpose else x
    if tp_group is not None:
        X = distributed_normalize_p2(work, eps, tp_group, normalize_in_double)
    else:
        X = _normalize(work, eps, normalize_in_double)
    coeffs = _schedule(steps, coefficient_type, custom_coefficient_sets)

    batched = X.ndim == 3
    step_name = "batched_newton_schulz_step" if batched else "newton_schulz_step"
    if medium:
        # torch has no float32-in / bf16-compute matmul, so the operands are rounded to bf16 explicitly.
        if use_syrk:
            if X.size(-1) % 8 or X.size(-2) % 8:
                _log_first_n(
                    logging.ERROR,
                    "syrk-skip",
                    8,
                    "[SYRK-SKIP] skipping SYRK for shape %s because GEMM M or N is not 16-byte aligned.",
                    tuple(X.shape),
                )
            else:
                step_name += "_tsyrk"
        X = X.to(torch.bfloat16)
        _log_first_n(logging.INFO, "bf16", 1, "Using BF16 I/O kernels for Newton-Schulz iteration.")

    for a, b, c in coeffs:
        # looked up per call so that a replaced module attribute takes effect
        X = globals()[step_name](X, a, b, c, tp_group=tp_group)

    X = X.to(torch.float32)
    if _out_scale != 1.0:
        X = X * _out_scale
    return X.mT if transpose else X


def newton_schulz_tp(
    x: torch.Tensor,
    steps: int,
    coefficient_type: NSCoeffT,
    tp_group: "torch.distributed.ProcessGroup",
    partition_dim: int | None = None,
    tp_mode: Literal["duplicated", "distributed"] = "duplicated",
    use_syrk: bool = False,
) -> torch.Tensor:
    """Newton-Schulz for a tensor sharded over ``tp_group`` along ``partition_dim`` (muon_utils.py:277-345).

    ``partition_dim=None`` means "not sharded": plain :func:`newton_schulz`.  ``"duplicated"`` gathers the
    shards, orthogonalises the full matrix on every rank and keeps the local slice.  ``"distributed"``
    keeps the shards in place, puts the sharded dimension on the contraction side and all-reduces the
    Gram matrix in every step.
    """
    if partition_dim is None:
        return newton_schulz(x, steps, coefficient_type, use_syrk=use_syrk)
    common: dict[str, Any] = dict(steps=steps, coefficient_type=coefficient_type, use_syrk=use_syrk)
    if tp_mode == "duplicated":
        world = tp_group.size()
        shards = [torch.empty_like(x) for _ in range(world)]
        torch.distributed.all_gather(shards, x, tp_group)
        full = newton_schulz(torch.cat(shards, dim=partition_dim), tp_group=None, **common)
        return full.chunk(world, dim=partition_dim)[tp_group.rank()]
    if tp_mode == "distributed":
        if partition_dim not in (0, 1):
            raise ValueError(f"Invalid partition_dim: {partition_dim}")
        return newton_schulz(x, transpose=(partition_dim == 0), tp_group=tp_group, **common)
    raise ValueError(f"Invalid tp_mode: {tp_mode}")


def _allreduce_gram(A: torch.Tensor, tp_group: Any) -> None:
    if tp_group is not None:
        torch.distributed.all_reduce(A, op=torch.distributed.ReduceOp.SUM, group=tp_group)


def _kernels_take(X: torch.Tensor) -> bool:
    """bf16 GPU operand of a step whose products the HIP kernels form: both dims multiples of 8 (16-byte rows),
    stored row-major or as its transpose.  Raises when such an operand arrives and ``libmi_ns.so`` is missing."""
    if not (hip_kernels.on_kernel_device(X) and X.dtype == torch.bfloat16 and X.numel() > 0):
        return False
    if X.size(-1) % 8 or X.size(-2) % 8 or not (X.is_contiguous() or X.mT.is_contiguous()):
        return False
    hip_kernels.require_library()
    return True


def _kernel_step(X: torch.Tensor, a: float, b: float, c: float, tp_group: Any) -> torch.Tensor:
    """One iteration on the HIP kernels, 2-D or batched: ``A = X X^T`` and ``B = c A A^T + b A`` on the
    lower-triangle kernel (``A`` is symmetric, so ``A A^T = A A``; the mirror image is written bit for bit), then
    ``a X + B X`` as one GEMM with the AXPY in its epilogue.  Three launches, each product accumulated in float32
    and rounded to bf16 once: the rounding points of ``X @ X.mT`` / ``addmm`` / ``baddbmm`` on bf16 operands."""
    syrk = triton_kernels.batched_tsyrk_ex if X.ndim == 3 else triton_kernels.tsyrk_ex
    A = syrk(X)
    _allreduce_gram(A, tp_group)
    if c == 0.0:
        return hip_kernels.gemm_axpy(A, X, alpha=b, beta=a)
    B = syrk(A, A, alpha=c, beta=b)
    return hip_kernels.gemm_axpy(B, X, alpha=1.0, beta=a)


def newton_schulz_step(X: torch.Tensor, a: float, b: float, c: float, tp_group: Any = None) -> torch.Tensor:
    """One iteration on a 2-D ``X``: ``a X + (b A + c A A) X`` (reference: muon_utils.py:348-378).

    ``c == 0`` takes the cubic form ``a X + b A X`` and skips the ``A A`` product.  With ``tp_group`` the Gram
    matrix is summed over the group, i.e. ``X`` is a shard along the contraction dimension.  bf16 GPU operands
    with both dims multiples of 8 run on the HIP kernels (:func:`_kernel_step`); any other device, dtype or shape
    on torch's matmuls, as in the reference.
    """
    if _kernels_take(X):
        return _kernel_step(X, a, b, c, tp_group)
    A = X @ X.mT
    _allreduce_gram(A, tp_group)
    if c == 0.0:
        return torch.addmm(X, A, X, alpha=b, beta=a)
    return torch.addmm(X, torch.addmm(A, A, A, alpha=c, beta=b), X, alpha=1.0, beta=a)


def batched_newton_schulz_step(X: torch.Tensor, a: float, b: float, c: float, tp_group: Any = None) -> torch.Tensor:
    """:func:`newton_schulz_step` for ``(B, M, N)`` input, every batch entry iterated independently (reference:
    muon_utils.py:381-411, ``baddbmm``); on the HIP kernels each product of the batch is one grouped launch."""
    if _kernels_take(X):
        return _kernel_step(X, a, b, c, tp_group)
    A = X @ X.mT
    _allreduce_gram(A, tp_group)
    if c == 0.0:
        return torch.baddbmm(X, A, X, alpha=b, beta=a)
    return torch.baddbmm(X, torch.baddbmm(A, A, A, alpha=c, beta=b), X, alpha=1.0, beta=a)


def _require_kernels() -> None:
    assert triton_kernels.HAS_TRITON_340, "the HIP kernel library (libmi_ns.so) is not available"


def newton_schulz_step_tsyrk(X: torch.Tensor, a: float, b: float, c: float, tp_group: Any = None) -> torch.Tensor:
    """One iteration on a 2-D bf16 ``X`` with the HIP kernels: two SYRKs (``X X^T`` and, ``A`` being symmetric,
    ``c A A^T + b A``) and one GEMM whose epilogue applies ``a X +``."""
    _require_kernels()
    return _kernel_step(X, a, b, c, tp_group)


def batched_newton_schulz_step_tsyrk(
    X: torch.Tensor, a: float, b: float, c: float, tp_group: Any = None
) -> torch.Tensor:
    """:func:`newton_schulz_step_tsyrk` for ``(B, M, N)`` bf16 input; each product is one grouped launch."""
    _require_kernels()
    return _kernel_step(X, a, b, c, tp_group)


_ORIGINAL_STEP_FNS = {
    "newton_schulz_step": newton_schulz_step,
    "batched_newton_schulz_step": batched_newton_schulz_step,
    "newton_schulz_step_tsyrk": newton_schulz_step_tsyrk,
    "batched_newton_schulz_step_tsyrk": batched_newton_schulz_step_tsyrk,
}
_ORIGINAL_NEWTON_SCHULZ = newton_schulz
