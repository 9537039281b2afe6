"""Batched bf16 SYRK ``d[b] = alpha * a[b] a[b]^T + beta * c[b]``: one grouped launch, grid = (tiles, batch).

Interface of the reference's ``batched_tsyrk_ex`` / ``can_use_batched_tsyrk``
(emerging_optimizers/triton_kernels/batched_syrk.py:237-363).
"""

from __future__ import annotations

import torch

from .. import _hip
from . import _launch


__all__ = ["batched_tsyrk_ex", "can_use_batched_tsyrk"]


def _layout_ok(t: torch.Tensor) -> bool:
    return t.is_contiguous() or t.mT.is_contiguous()


def can_use_batched_tsyrk(a: torch.Tensor, c: torch.Tensor | None = None) -> bool:
    """Whether :func:`batched_tsyrk_ex` accepts these operands (so callers can pick ``torch.baddbmm`` instead).

    Requirements: kernels loadable, GPU tensor, bf16, 3-D, ``a`` or ``a.mT`` contiguous, N and K multiples
    of 8 (16-byte vector loads), and a matching, contiguous-either-way ``c`` if one is given.
    """
    if not _hip.available() or not a.is_cuda or a.dtype != torch.bfloat16 or a.dim() != 3:
        return False
    if not _layout_ok(a):
        return False
    b, n, k = a.shape
    if n % 8 or k % 8:
        return False
    if c is not None:
        if tuple(c.shape) != (b, n, n) or c.dtype != a.dtype or not _layout_ok(c):
            return False
    return True


def batched_tsyrk_ex(
    a: torch.Tensor,
    c: torch.Tensor | None = None,
    alpha: float = 1.0,
    beta: float = 0.0,
    skip_upper_triangle: bool = False,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Stand-in for ``torch.baddbmm(c, a, a.mT, beta=beta, alpha=alpha)`` that computes lower-triangle tiles only.

    ``a``: (B, N, K) bf16 with ``a`` or ``a.mT`` contiguous; each ``c[b]`` symmetric.  Returns (B, N, N) bf16,
    every matrix bitwise symmetric (unless ``skip_upper_triangle``).
    """
    if not _hip.available():
        raise RuntimeError("HIP kernels are unavailable: libmi_ns.so could not be loaded")
    if a.dtype != torch.bfloat16:
        raise TypeError("Input tensor must be bfloat16")
    if a.dim() != 3:
        raise TypeError("Input tensor must be 3D of shape (B, N, K)")
    if not _layout_ok(a):
        raise TypeError("invalid input tensor layout. a or a.mT must be contiguous.")
    batch, n, k = a.shape
    if n % 8 or k % 8:
        raise RuntimeError(f"N and K must be multiples of 8 for 16-byte bf16 loads, got N={n}, K={k}")
    c_ok = (c is None and beta == 0.0) or (c is not None and tuple(c.shape) == (batch, n, n))
    if not c_ok:
        raise RuntimeError("if c is provided, c must be of shape (B, N, N)")
    if c is not None and not _layout_ok(c):
        raise RuntimeError("if c is provided, c or c.mT must be contiguous")
    if out is None:
        d = torch.empty((batch, n, n), device=a.device, dtype=a.dtype)
    else:
        if tuple(out.shape) != (batch, n, n) or out.dtype != a.dtype or out.device != a.device:
            raise RuntimeError("out must be same shape/device/dtype as output")
        if not out.is_contiguous():
            raise RuntimeError("out must be contiguous")
        d = out
    _launch.require_gpu(a, "batched_tsyrk_ex")
    a_trans = not a.is_contiguous()
    mem_a = a.mT if a_trans else a
    c_mem = None
    if beta != 0.0:
        if c.dtype != a.dtype or c.device != a.device:
            raise RuntimeError("c must have the dtype and device of a")
        c_mem = c if c.is_contiguous() else c.mT
    _launch.syrk_launch(mem_a, a_trans, batch, n, k, c_mem, alpha, beta, d, skip_upper_triangle)
    return d
