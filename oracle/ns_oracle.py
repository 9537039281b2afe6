"""CPU oracle for the Muon orthogonalisation path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A plain numpy restatement of what NVIDIA-NeMo/Emerging-Optimizers computes on this path.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it; the
package under ``emerging-optimizers_amd/`` never does.

Every function cites the reference lines it follows (paths relative to the reference checkout).
How each one is pinned (``tests/test_oracle.py``):

* coefficient tables        -- literal constants; fixed-point identities p(1) of three tables
* coefficient_iterator      -- closed form ``sets[i % L]`` / ``sets[min(i, L-1)]``
* newton_schulz (fp32/fp64) -- SVD closed form: singular vectors are invariant, singular values follow
                               the scalar recurrence ``s <- a s + b s^3 + c s^5`` (``svd_polynomial``)
* newton_schulz_step        -- same closed form with one step; cubic case against ``a x + b (x x^T) x``
* syrk / gemm_axpy          -- brute-force Python loops on tiny integer inputs (exact arithmetic)
* round_to_bf16             -- exhaustive comparison with the IEEE definition on a value sweep incl. ties
* muon_scale_factor         -- ``math.sqrt`` closed forms
* optimizer step            -- equals textbook SGD / SGD-with-momentum updates on integer data
* tri_decode                -- brute-force bijection onto ``{(i, j): j <= i < T}``

The reference itself holds no stored golden vectors for this path (all of its expectations are computed at
test time), so the checks above are what anchors this file.
"""

from __future__ import annotations

import itertools
import math
from typing import Iterator, Sequence

import numpy as np


# --------------------------------------------------------------------------------------------
# Coefficient tables: emerging_optimizers/orthogonalized_optimizers/muon_utils.py:30-90 (data).
# --------------------------------------------------------------------------------------------
COEFFICIENT_SETS: dict[str, list[tuple[float, float, float]]] = {
    "simple": [(3.4445, -4.7750, 2.0315)],
    "quintic": [
        (4.0848, -6.8946, 2.9270),
        (3.9505, -6.3029, 2.6377),
        (3.7418, -5.5913, 2.3037),
        (2.8769, -3.1427, 1.2046),
        (2.8366, -3.0525, 1.2012),
    ],
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
    "cans": [
        (8.4703, -25.1081, 18.6293),
        (4.1828, -3.1087, 0.5806),
        (3.9619, -2.9541, 0.5630),
        (3.2866, -2.4647, 0.5074),
        (2.2737, -1.6447, 0.4162),
    ],
    "aol": [
        (4.0098, -7.0585, 2.4635),
        (3.4585, -5.5479, 2.5959),
        (2.7573, -3.2939, 1.4254),
        (2.7215, -3.0494, 1.3169),
    ],
    "deepseekv4": [(3.4445, -4.7750, 2.0315)] * 8 + [(2.0, -1.5, 0.5)] * 2,
    "cubic5": [
        (3.3656576, -3.3420992, 0.0),
        (2.5744352, -1.4957376, 0.0),
        (2.5368962, -1.4312570, 0.0),
        (2.4418906, -1.2764040, 0.0),
        (2.2230472, -0.9630650, 0.0),
    ],
}

# muon_utils.py:239-240: these families keep repeating their last tuple, the others cycle.
REPEAT_LAST_TYPES = ("polar_express", "cans", "deepseekv4")


def coefficient_iterator(steps: int, sets: Sequence[tuple[float, float, float]], mode: str = "cycle") -> Iterator:
    """muon_utils.py:93-129.  ``cycle``: sets[i % L]; ``repeat_last``: sets[min(i, L-1)]."""
    if not sets:
        raise ValueError("coefficient_sets must be non-empty.")
    if mode not in ("cycle", "repeat_last"):
        raise ValueError(f"Invalid mode: {mode}. Expected 'cycle' or 'repeat_last'.")
    n = len(sets)
    for i in range(steps):
        yield sets[i % n] if mode == "cycle" else sets[min(i, n - 1)]


def expand_coefficients(steps: int, coefficient_type: str, custom=None) -> list[tuple[float, float, float]]:
    """Table lookup + iteration mode of muon_utils.py:224-241 as a flat list of ``steps`` tuples."""
    if coefficient_type in COEFFICIENT_SETS:
        sets = COEFFICIENT_SETS[coefficient_type]
    elif coefficient_type == "custom":
        if custom is None:
            raise ValueError("custom_coefficient_sets must be provided when coefficient_type is 'custom'.")
        sets = custom
    else:
        raise ValueError(f"Invalid coefficient type: {coefficient_type}")
    if coefficient_type == "cubic5" and steps != len(sets):
        raise ValueError(f"cubic5 is a fixed {len(sets)}-step schedule; got steps={steps}. Use steps=5.")
    mode = "repeat_last" if coefficient_type in REPEAT_LAST_TYPES else "cycle"
    return list(coefficient_iterator(steps, sets, mode))


# --------------------------------------------------------------------------------------------
# bfloat16 emulation (numpy has no bf16): round-to-nearest-even on the upper 16 bits of float32.
# --------------------------------------------------------------------------------------------
def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32.  NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    out = rounded.astype(np.uint32).view(np.float32).reshape(x.shape)
    return np.where(np.isnan(x), x, out)


def _mT(x: np.ndarray) -> np.ndarray:
    return np.swapaxes(x, -1, -2)


# --------------------------------------------------------------------------------------------
# SYRK and the AXPY-GEMM as the reference defines them.
# --------------------------------------------------------------------------------------------
def syrk(a: np.ndarray, c: np.ndarray | None = None, alpha: float = 1.0, beta: float = 0.0) -> np.ndarray:
    """``bf16(alpha * a a^T + beta * c)`` with float32 accumulation and float32 epilogue.

    triton_kernels/syrk.py:198-215 (2-D) and triton_kernels/batched_syrk.py:203-224 (batched): the product
    is accumulated in float32, scaled by alpha, beta*c added in float32, then rounded once to bf16.
    ``a`` holds bf16-representable float32 values; the result is returned as float32 holding bf16 values.
    """
    a = np.asarray(a, dtype=np.float32)
    acc = np.matmul(a, _mT(a))
    acc = np.float32(alpha) * acc
    if beta != 0.0:
        acc = np.float32(beta) * np.asarray(c, dtype=np.float32) + acc
    return round_to_bf16(acc)


def gemm_axpy(bm: np.ndarray, x: np.ndarray, alpha: float, beta: float, *, round_bf16: bool = True) -> np.ndarray:
    """``beta * x + alpha * (bm @ x)``: torch.addmm(X, B, X, alpha=alpha, beta=beta) of muon_utils.py:374-377."""
    acc = np.matmul(np.asarray(bm, dtype=np.float32), np.asarray(x, dtype=np.float32))
    out = np.float32(beta) * np.asarray(x, dtype=np.float32) + np.float32(alpha) * acc
    return round_to_bf16(out) if round_bf16 else out


# --------------------------------------------------------------------------------------------
# Newton-Schulz.
# --------------------------------------------------------------------------------------------
def frobenius_normalize(x: np.ndarray, eps: float = 1e-15, in_double: bool = False) -> np.ndarray:
    """muon_utils.py:212-222.  float32: x / max(||x||_F, eps).  double: x / float32(||x||_F) with no clamp."""
    x = np.asarray(x, dtype=np.float32)
    if in_double:
        norm = np.sqrt(np.sum(x.astype(np.float64) ** 2, axis=(-2, -1), keepdims=True)).astype(np.float32)
        return x / norm
    norm = np.sqrt(np.sum(x * x, axis=(-2, -1), keepdims=True, dtype=np.float32))
    return x / np.maximum(norm, np.float32(eps))


def newton_schulz_step(x: np.ndarray, a: float, b: float, c: float, *, bf16: bool = False) -> np.ndarray:
    """One iteration, muon_utils.py:348-378 (and its batched / SYRK twins :381-476).

    ``A = X X^T``; quintic (c != 0): ``B = b A + c A A``, ``X' = a X + B X``; cubic (c == 0): ``X' = a X + b A X``.
    With ``bf16=True`` every product is rounded to bf16 after a float32 epilogue, which is what the reference
    executes under matmul precision "medium" (X, A and B are bf16 tensors there).
    """
    dt = x.dtype
    if bf16:
        gram = syrk(x)
        if c != 0.0:
            poly = syrk(gram, gram, alpha=c, beta=b)
            return gemm_axpy(poly, x, 1.0, a)
        return gemm_axpy(gram, x, b, a)
    gram = np.matmul(x, _mT(x))
    if c != 0.0:
        poly = dt.type(b) * gram + dt.type(c) * np.matmul(gram, gram)
        return dt.type(a) * x + np.matmul(poly, x)
    return dt.type(a) * x + dt.type(b) * np.matmul(gram, x)


def newton_schulz(
    x: np.ndarray,
    steps: int,
    coefficient_type: str = "quintic",
    custom_coefficient_sets=None,
    eps: float = 1e-15,
    transpose: bool | None = None,
    normalize_in_double: bool = False,
    precision: str = "highest",
    compute_dtype=np.float32,
) -> np.ndarray:
    """muon_utils.py:149-274 on one process (tp_group=None).

    precision "highest": float32 (or ``compute_dtype``) arithmetic throughout.
    precision "medium" : the reference's bf16 schedule (:245-269): normalise in float32, round X to bf16,
    iterate with bf16-rounded products, return float32.
    """
    x = np.asarray(x)
    if x.ndim < 2 or x.ndim > 3:
        raise TypeError(f"Input tensor x must be 2d or 3d (batched 2d), got {x.ndim}d")
    if x.dtype != np.float32:
        raise TypeError(f"Input tensor x must be in float32, got {x.dtype}")
    if transpose is None:
        transpose = x.shape[-2] > x.shape[-1]
    if transpose:
        x = _mT(x)
    X = frobenius_normalize(x, eps, normalize_in_double)
    coeffs = expand_coefficients(steps, coefficient_type, custom_coefficient_sets)
    bf16 = precision == "medium"
    if bf16:
        X = round_to_bf16(X)
    else:
        X = X.astype(compute_dtype)
    for a, b, c in coeffs:
        X = newton_schulz_step(X, a, b, c, bf16=bf16)
    X = X.astype(np.float32)
    return _mT(X) if transpose else X


def group_schedule(coeffs: Sequence[tuple[float, float, float]], mode: int) -> list[int]:
    """Group sizes of the single-call GPU driver: g = g steps on one Gram matrix, 1 = an ordinary step.

    ``mode`` 0: all ones.  1: pairs alternate with single steps, starting with a pair (5 steps: 2 + 1 + 2); a pair needs quintic
    coefficients (c != 0) in both of its steps.  2: as 1, but the first three steps form one group when at least
    two more steps follow, all three are quintic and ``(a_1 a_2)**2 <= 400`` (the factor by which the rounding
    noise of the first Gram matrix has grown in the third); 5 steps: 3 + 2.
    """
    groups, s, want_group = [], 0, True
    quintic = lambda k: coeffs[k][2] != 0.0
    while s < len(coeffs):
        size = 1
        if mode and want_group and s + 1 < len(coeffs) and quintic(s) and quintic(s + 1):
            size = 2
            if mode == 2 and s == 0 and len(coeffs) >= 5 and quintic(2) and (coeffs[0][0] * coeffs[1][0]) ** 2 <= 400.0:
                size = 3
        groups.append(size)
        s += size
        want_group = size != 2  # a pair is followed by a single step; the opening triple may be followed by a pair
    return groups


def pair_schedule(coeffs: Sequence[tuple[float, float, float]], pairs: bool) -> list[int]:
    """:func:`group_schedule` restricted to pairs (mode 1) or single steps (mode 0)."""
    return group_schedule(coeffs, 1 if pairs else 0)


def _mirror_lower(mat: np.ndarray) -> np.ndarray:
    """What the lower-triangle kernels store: the computed lower triangle and its mirror image."""
    return np.tril(mat) + _mT(np.tril(mat, -1))


def newton_schulz_shifted_bf16(
    x: np.ndarray,
    steps: int,
    coefficient_type: str = "quintic",
    custom_coefficient_sets=None,
    eps: float = 1e-15,
    normalize_in_double: bool = False,
    pairs: bool | int | None = None,
) -> np.ndarray:
    """CPU model of the rounding schedule of the single-call GPU driver (``mi_newton_schulz_bf16``).

    Not a restatement of the reference: the reference rounds X, A = X X^T and B = b A + c A^2 to bf16 in every
    step (muon_utils.py:262, 414-476), which leaves it 1.0e-2 .. 1.3e-2 (relative Frobenius) away from its own
    float32 path because bf16 rounding of the O(1) diagonal of A dominates.  The driver stores A' = A - s I
    with s = ||X||_F^2 / m instead and folds the identity part into the epilogue scalars
        B' = c A'^2 + (b + 2 c s) A',      X' = (a + b s + c s^2) X + B' X,
    which is algebraically the same iteration for any s.  The last step is written to float32 unrounded.
    The input is rounded to bf16 before the division by the norm, which then enters the first products as a
    scalar (one pass over the float32 input instead of two).

    For wide matrices (m >= 1024 and n >= 2 m, or the short, very wide per-head shapes whose Gram matrix is summed
    from K slices; ``pairs`` = False / True / 2 overrides the rule with mode 0 / 1 / 2 of :func:`group_schedule`)
    the driver takes steps two -- at the start, for the large shapes, three -- at a time
    on one Gram matrix.  All factors are polynomials of A and commute, so with A_k = s_k I + D_k,
    q_k = e_k I + R_k (R_k = B' of step k, e_k = a_k + b_k s_k + c_k s_k^2) and the accumulated multiplier
    q_k ... q_1 = alpha_k I + S_k:
        T'_k = R_k D_k + e_k D_k + s_k R_k,  D_{k+1} = R_k T'_k + e_k T'_k + e_k s_k R_k,  s_{k+1} = e_k^2 s_k,
        S_k = R_k S_{k-1} + e_k S_{k-1} + alpha_{k-1} R_k  (S_1 = R_1),  alpha_k = e_1 ... e_k,
        X' = alpha_g X + S_g X  after the g steps of the group,
    each m x m product computed on its lower triangle, mirrored and rounded to bf16.
    This function reproduces those rounding points so that GPU results can be compared tightly.
    """
    x = np.asarray(x)
    if x.dtype != np.float32 or x.ndim not in (2, 3):
        raise TypeError("float32 2-D or 3-D input expected")
    transpose = x.shape[-2] > x.shape[-1]
    if transpose:
        x = _mT(x)
    f = np.float32
    m, n = x.shape[-2:]
    coeffs = expand_coefficients(steps, coefficient_type, custom_coefficient_sets)
    # The input is cast to bf16 unnormalised and 1 / ||x||_F enters the first group's products (r^2 in the Gram
    # matrix, r in X' = ...).  The deferral is limited to norms whose squares are safe in float32.
    if normalize_in_double:
        norm = np.sqrt(np.sum(x.astype(np.float64) ** 2, axis=(-2, -1), keepdims=True)).astype(np.float32)
    else:
        norm = np.maximum(np.sqrt(np.sum(x * x, axis=(-2, -1), keepdims=True, dtype=np.float32)), f(eps))
    deferred = len(coeffs) > 0 and bool(np.all((norm >= f(1e-10)) & (norm <= f(1e10))))
    if deferred:
        X = round_to_bf16(x)
        r = f(1.0) / norm
        sumsq = (np.sqrt(np.sum(x * x, axis=(-2, -1), keepdims=True, dtype=np.float32)) / norm) ** 2
    else:
        X = round_to_bf16(frobenius_normalize(x, eps, normalize_in_double))
        r = np.ones_like(norm)
        sumsq = np.ones(X.shape[:-2] + (1, 1), dtype=np.float32)
    if pairs is None:
        batch = int(np.prod(x.shape[:-2])) if x.ndim == 3 else 1
        split_k_gram = m % 128 == 0 and m <= 256 and n % 512 == 0 and n >= 1024 and batch * (n // 512) <= 65535
        mode = 2 if (split_k_gram or (m >= 1024 and n >= 2 * m)) else 0
    else:
        mode = int(pairs)  # False / True / 2
    eye = np.eye(m, dtype=np.float32)
    done = 0
    for group in group_schedule(coeffs, mode):
        a, b, c = (f(v) for v in coeffs[done])
        s = sumsq / f(m)
        gram = round_to_bf16((r * r) * np.matmul(X, _mT(X)) - s * eye)
        if group == 1 and c == 0.0:
            Xn = ((a + b * s) * r) * X + (b * r) * np.matmul(gram, X)
        else:
            # A_k = s_k I + D_k;  accumulated multiplier alpha I + S
            D, sk, alpha, S = gram, s, f(1.0), None
            for k in range(group):
                ak, bk, ck = (f(v) for v in coeffs[done + k])
                R = round_to_bf16(ck * np.matmul(D, D) + (bk + f(2.0) * ck * sk) * D)
                e = ak + bk * sk + ck * sk * sk
                S = R if k == 0 else round_to_bf16(_mirror_lower(np.matmul(R, S) + e * S + alpha * R))
                if k + 1 < group:
                    T = round_to_bf16(_mirror_lower(np.matmul(R, D) + e * D + sk * R))
                    D = round_to_bf16(_mirror_lower(np.matmul(R, T) + e * T + (e * sk) * R))
                    sk = e * e * sk
                alpha = alpha * e
            Xn = (alpha * r) * X + r * np.matmul(S, X)
        done += group
        r = np.ones_like(norm)  # from here on X is normalised
        sumsq = np.sum(Xn * Xn, axis=(-2, -1), keepdims=True, dtype=np.float32)
        X = Xn if done == len(coeffs) else round_to_bf16(Xn)
    X = X.astype(np.float32)
    return _mT(X) if transpose else X


def svd_polynomial(x: np.ndarray, coeffs: Sequence[tuple[float, float, float]], eps: float = 1e-15) -> np.ndarray:
    """Closed form of the iteration in float64, independent of any matrix-product code path.

    With x / ||x||_F = U diag(s) V^T, one step maps it to U diag(a s + b s^3 + c s^5) V^T, because
    X X^T = U diag(s^2) U^T.  So the result of the whole schedule is U diag(p_k(...p_1(s))) V^T.
    """
    x = np.asarray(x, dtype=np.float64)
    transpose = x.shape[-2] > x.shape[-1]
    if transpose:
        x = _mT(x)
    x = x / max(np.linalg.norm(x), eps)
    u, s, vt = np.linalg.svd(x, full_matrices=False)
    for a, b, c in coeffs:
        s = a * s + b * s**3 + c * s**5
    out = (u * s) @ vt
    return _mT(out) if transpose else out


# --------------------------------------------------------------------------------------------
# Muon pieces around the iteration.
# --------------------------------------------------------------------------------------------
def muon_scale_factor(size_out: int, size_in: int, mode: str = "spectral") -> float:
    """orthogonalized_optimizers/muon.py:190-216."""
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "spectral":
        return max(size_out, size_in) ** 0.5
    if mode == "unit_rms_norm":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for Muon update scale factor: {mode}")


def optimizer_step(
    p: np.ndarray,
    grad: np.ndarray,
    momentum_buffer: np.ndarray,
    *,
    lr: float,
    momentum: float,
    weight_decay: float,
    weight_decay_method: str = "decoupled",
    nesterov: bool = False,
    orthogonalize=lambda g: g,
) -> tuple[np.ndarray, np.ndarray]:
    """One parameter update of OrthogonalizedOptimizer.step, orthogonalized_optimizer.py:164-212 with the
    weight-decay variants of mixin.py:43-56.  Returns ``(new_p, new_momentum_buffer)``; float32 throughout."""
    f = np.float32
    p = np.asarray(p, dtype=np.float32).copy()
    grad = np.asarray(grad, dtype=np.float32).copy()
    buf = np.asarray(momentum_buffer, dtype=np.float32).copy()
    if weight_decay != 0.0:
        if weight_decay_method == "decoupled":
            p = p + f(-weight_decay * lr) * p
        elif weight_decay_method == "independent":
            p = p + f(-weight_decay) * p
        elif weight_decay_method == "l2":
            grad = grad + f(weight_decay) * p
        elif weight_decay_method == "palm":
            p = p + f(-(weight_decay * lr * lr)) * p
        else:
            raise ValueError(f"Invalid weight decay method: {weight_decay_method}")
    # lerp_(grad, 1 - momentum): buf + w (grad - buf)
    buf = buf + f(1 - momentum) * (grad - buf)
    g = grad + f(momentum) * (buf - grad) if nesterov else buf
    update = np.asarray(orthogonalize(g), dtype=np.float32)
    p = p + f(-lr) * update
    return p, buf


def muon_orthogonalize(grad, *, steps=5, coefficient_type="quintic", scale_mode="spectral", extra_scale_factor=1.0,
                       precision="medium"):
    """Muon's closure, muon.py:117-132: newton_schulz(grad) * scale_factor * extra_scale_factor."""
    orth = newton_schulz(grad, steps, coefficient_type, precision=precision)
    scale = muon_scale_factor(grad.shape[-2], grad.shape[-1], scale_mode)
    return orth * np.float32(scale) * np.float32(extra_scale_factor)


# --------------------------------------------------------------------------------------------
# Lower-triangle tile enumeration used by the triangular launch grids.
# --------------------------------------------------------------------------------------------
def tri_decode(pid: int) -> tuple[int, int]:
    """Linear tile id -> (i, j), j <= i: i = floor((sqrt(8 pid + 1) - 1) / 2), j = pid - i (i + 1) / 2
    (triton_kernels/syrk.py:285-291, batched_syrk.py:185-193), evaluated with exact integer arithmetic."""
    i = (math.isqrt(8 * pid + 1) - 1) // 2
    return i, pid - i * (i + 1) // 2


def flops_sym(m: int, n: int, steps: int, batch: int = 1) -> int:
    """Symmetric-halved FLOP count of ``steps`` quintic iterations on a batch of (m, n), m <= n."""
    return batch * steps * (3 * m * m * n + m**3)


__all__ = [name for name in dir() if not name.startswith("_") and name not in ("itertools", "math", "np")]


def tri_block_decode(s: int, T: int, block: int = 6) -> tuple[int, int]:
    """Blocked enumeration of the lower-triangle tiles used by the XCD-aware SYRK launch (build-specific, no
    counterpart in the reference): block-rows of ``block`` tile rows; inside a block-row the full
    ``block``-wide rectangles first (row-major), then the triangular block on the diagonal."""
    r = (math.isqrt(8 * s + 1) - 1) // 2
    bi = r // block
    row0 = bi * block
    h = min(block, T - row0)
    u = s - row0 * (row0 + 1) // 2
    rect = h * block
    if u < bi * rect:
        bj, v = divmod(u, rect)
        return row0 + v // block, bj * block + v % block
    u -= bi * rect
    lr = (math.isqrt(8 * u + 1) - 1) // 2
    return row0 + lr, row0 + (u - lr * (lr + 1) // 2)
