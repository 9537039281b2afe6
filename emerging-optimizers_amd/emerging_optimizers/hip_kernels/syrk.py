"""2-D bf16 SYRK: ``D = alpha * A A^T + beta * C`` on the gfx950 tile engine.

Interface of the reference's ``tsyrk_ex`` / ``tsyrk_ex_small_matrix``
(emerging_optimizers/triton_kernels/syrk.py:335-408, 411-500): same arguments, same exception types
and messages.  The reference needs two Triton kernels (rectangular grid with early exit, triangular
grid); here both names reach the same HIP kernel, which always launches lower-triangle tiles only.
"""

from __future__ import annotations

import torch

from . import _launch


__all__ = ["tsyrk_ex", "tsyrk_ex_small_matrix"]


def _validate(a: torch.Tensor, c: torch.Tensor | None, beta: float) -> tuple[int, int]:
    if a.dtype != torch.bfloat16:
        raise TypeError("Input tensor must be bfloat16")
    if a.dim() != 2:
        raise TypeError("Input tensor must be 2D")
    if not (a.is_contiguous() or a.T.is_contiguous()):
        raise TypeError("invalid input tensor layout. a or a.T must be contiguous.")
    n, k = a.shape
    c_ok = (c is None and beta == 0.0) or (c is not None and tuple(c.shape) == (n, n))
    if not c_ok:
        raise RuntimeError("if c is provided, c must be of shape (N, N)")
    if c is not None and not (c.is_contiguous() or c.T.is_contiguous()):
        raise RuntimeError("if c is provided, c or c.T must be contiguous")
    return n, k


def _run(a, c, alpha, beta, skip_upper_triangle, out) -> torch.Tensor:
    n, k = _validate(a, c, beta)
    if out is None:
        d = torch.empty((n, n), device=a.device, dtype=a.dtype)
    else:
        if tuple(out.shape) != (n, n) or out.dtype != a.dtype or out.device != a.device:
            raise RuntimeError("out must be same shape/device/dtype as output")
        if not out.is_contiguous():
            raise RuntimeError("out must be contiguous")
        d = out
    _launch.require_gpu(a, "tsyrk_ex")
    # A 1-row/1-column operand is contiguous both ways; prefer the plain layout then.
    a_trans = not a.is_contiguous()
    mem_a = a.T if a_trans else a
    c_mem = None
    if beta != 0.0:
        if c.dtype != a.dtype or c.device != a.device:
            raise RuntimeError("c must have the dtype and device of a")
        # C is symmetric, so whichever orientation is contiguous can be read as-is.
        c_mem = c if c.is_contiguous() else c.T
    _launch.syrk_launch(mem_a, a_trans, 1, n, k, c_mem, alpha, beta, d, skip_upper_triangle)
    return d


def tsyrk_ex(
    a: torch.Tensor,
    c: torch.Tensor | None = None,
    alpha: float = 1.0,
    beta: float = 0.0,
    skip_upper_triangle: bool = False,
) -> torch.Tensor:
    """``alpha * a @ a.T + beta * c`` for bf16 ``a`` of shape (N, K); ``c`` must be symmetric.

    float32 accumulation, one rounding to bf16.  With ``skip_upper_triangle`` the strictly upper
    tiles of the result are left unwritten.  The result is otherwise bitwise symmetric.
    """
    return _run(a, c, alpha, beta, skip_upper_triangle, None)


def tsyrk_ex_small_matrix(
    a: torch.Tensor,
    c: torch.Tensor | None = None,
    alpha: float = 1.0,
    beta: float = 0.0,
    skip_upper_triangle: bool = False,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Same operation as :func:`tsyrk_ex` with an optional preallocated ``out`` (N, N) bf16 tensor."""
    return _run(a, c, alpha, beta, skip_upper_triangle, out)
