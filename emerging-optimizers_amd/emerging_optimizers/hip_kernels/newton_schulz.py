"""GEMM+AXPY and the single-call Newton-Schulz driver of libmi_ns.so."""

from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from .. import _hip
from . import _launch


__all__ = ["gemm_axpy", "fused_newton_schulz", "fused_supported", "fused_muon_update", "on_kernel_device", "require_library"]


def require_library() -> None:
    """Raises ``RuntimeError`` unless ``libmi_ns.so`` is loaded: GPU operands that the kernels serve never take
    another path silently."""
    _hip.lib()


def on_kernel_device(t: torch.Tensor) -> bool:
    """``t`` lives on a gfx950 GPU, the only part the kernels are compiled for.  Tensors on any other GPU stay on
    torch's own operators, as the reference does for GPUs that its kernels do not support (muon.py:101-115)."""
    return t.is_cuda and _hip.device_is_gfx950(t.device)


def gemm_axpy(
    bm: torch.Tensor,
    x: torch.Tensor,
    alpha: float = 1.0,
    beta: float = 1.0,
    *,
    out_dtype: torch.dtype = torch.bfloat16,
    out_scale: float = 1.0,
) -> torch.Tensor:
    """``beta * x + alpha * (bm @ x)`` for bf16 ``bm`` (.., m, m) and ``x`` (.., m, n), 2-D or batched 3-D.

    The HIP counterpart of ``torch.addmm(X, B, X, alpha=alpha, beta=beta)`` / ``torch.baddbmm`` in a
    Newton-Schulz step (muon_utils.py:374-377, 407-410 of the reference).  ``x`` or ``x.mT`` must be
    contiguous; the result has the layout of ``x``.  ``out_dtype=torch.float32`` returns
    ``out_scale * (...)`` without the intermediate bf16 rounding.
    """
    if bm.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise TypeError("gemm_axpy operands must be bfloat16")
    if x.dim() not in (2, 3) or bm.dim() != x.dim():
        raise TypeError("gemm_axpy operands must both be 2D or both be 3D")
    _launch.require_gpu(x, "gemm_axpy")
    batch = x.shape[0] if x.dim() == 3 else 1
    m, n = x.shape[-2], x.shape[-1]
    if tuple(bm.shape[-2:]) != (m, m) or (x.dim() == 3 and bm.shape[0] != batch):
        raise RuntimeError(f"bm must be of shape (..., {m}, {m}), got {tuple(bm.shape)}")
    if not (x.is_contiguous() or x.mT.is_contiguous()):
        raise TypeError("invalid input tensor layout. x or x.mT must be contiguous.")
    if m % 8 or n % 8:
        raise RuntimeError(f"M and N must be multiples of 8 for 16-byte bf16 loads, got M={m}, N={n}")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("out_dtype must be bfloat16 or float32")
    bm = bm.contiguous()
    x_trans = not x.is_contiguous()
    mem_x = x.mT if x_trans else x
    out_mem = torch.empty(mem_x.shape, device=x.device, dtype=out_dtype)
    lib = _hip.lib()
    with torch.cuda.device(x.device):
        rc = lib.mi_gemm_axpy_bf16(
            _launch.ptr(bm), m * m, m,
            _launch.ptr(mem_x), m * n, mem_x.shape[-1], int(x_trans),
            _launch.ptr(out_mem), m * n, mem_x.shape[-1],
            batch, m, n, float(alpha), float(beta),
            int(out_dtype == torch.float32), float(out_scale), _hip.current_stream_ptr(x.device),
        )  # fmt: skip
    _hip.check(rc)
    return out_mem.mT if x_trans else out_mem


def fused_supported(x: torch.Tensor) -> bool:
    """True when :func:`fused_newton_schulz` can take ``x``: GPU float32, 2-D/3-D, both dims multiples of 8.
    Raises ``RuntimeError`` for such a tensor when ``libmi_ns.so`` is missing (no silent slow path on the GPU)."""
    if not (
        on_kernel_device(x)
        and x.dtype == torch.float32
        and x.dim() in (2, 3)
        and x.shape[-1] % 8 == 0
        and x.shape[-2] % 8 == 0
        and x.numel() > 0
    ):
        return False
    require_library()
    return True


def frob_normalize(
    x: torch.Tensor,
    eps: float = 1e-7,
    *,
    normalize_in_double: bool = False,
    out_dtype: torch.dtype = torch.float32,
    return_norm: bool = False,
):
    """``x / max(||x||_F, eps)`` per matrix of a float32 tensor whose last two dimensions are the matrix (the
    pre-normalisation of ``newton_schulz``, muon_utils.py:212-222): squares summed in float32 like
    ``torch.nn.functional.normalize`` or, with ``normalize_in_double``, in float64 (the reference's hook for
    ill-scaled inputs); result in float32 or bfloat16.  One ``mi_frob_normalize`` call.  With ``return_norm`` also the
    divisor used per matrix (float32, on the device)."""
    if not x.is_cuda or x.dtype != torch.float32:
        raise RuntimeError("frob_normalize needs a float32 tensor on the GPU")
    if x.dim() < 2 or not x.is_contiguous():
        raise ValueError("frob_normalize needs a contiguous tensor of at least two dimensions")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("out_dtype must be float32 or bfloat16")
    numel = x.shape[-2] * x.shape[-1]
    batch = x.numel() // numel if numel else 0
    out = torch.empty_like(x, dtype=out_dtype)
    norm = torch.empty(max(batch, 1), device=x.device, dtype=torch.float32)
    if batch == 0:
        return (out, norm[:0]) if return_norm else out
    lib = _hip.lib()
    with torch.cuda.device(x.device):
        partials = torch.empty(lib.mi_frob_partials_len(batch, numel), device=x.device, dtype=torch.float64)
        rc = lib.mi_frob_normalize(
            _launch.ptr(x), batch, numel, float(eps), int(bool(normalize_in_double)), _launch.ptr(out),
            int(out_dtype == torch.bfloat16), _launch.ptr(partials), _launch.ptr(norm), _hip.current_stream_ptr(x.device),
        )  # fmt: skip
    _hip.check(rc)
    return (out, norm[:batch]) if return_norm else out


def fused_newton_schulz(
    x: torch.Tensor,
    coefficients: Sequence[tuple[float, float, float]],
    eps: float = 1e-15,
    normalize_in_double: bool = False,
    out_scale: float = 1.0,
) -> torch.Tensor:
    """Normalise, iterate and rescale in one library call; returns a new float32 tensor shaped like ``x``.

    Covers the "medium"-precision body of the reference's ``newton_schulz`` (muon_utils.py:212-273) for one
    process.  The iteration runs on the orientation with the shorter leading dimension, read in place.
    """
    if not fused_supported(x):
        raise RuntimeError(f"fused_newton_schulz cannot take a {x.dtype} tensor of shape {tuple(x.shape)} on {x.device}")
    xc = x if x.is_contiguous() else x.contiguous()
    batch = xc.shape[0] if xc.dim() == 3 else 1
    rows, cols = xc.shape[-2], xc.shape[-1]
    out = torch.empty_like(xc)
    lib = _hip.lib()
    steps = len(coefficients)
    flat = [float(v) for abc in coefficients for v in abc]
    abc = (ctypes.c_float * max(1, len(flat)))(*flat)
    with torch.cuda.device(x.device):
        nbytes = lib.mi_newton_schulz_workspace_bytes(batch, rows, cols)
        ws = _launch.workspace(x.device, nbytes)
        rc = lib.mi_newton_schulz_bf16(
            _launch.ptr(xc), _launch.ptr(out), batch, rows, cols, abc, steps, float(eps),
            int(bool(normalize_in_double)), float(out_scale), _launch.ptr(ws), ws.numel(),
            _hip.current_stream_ptr(x.device),
        )  # fmt: skip
    _hip.check(rc)
    return out


def fused_muon_update(
    param: torch.Tensor,
    grad: torch.Tensor,
    momentum_buffer: torch.Tensor,
    coefficients: Sequence[tuple[float, float, float]],
    *,
    beta: float,
    nesterov: bool,
    param_decay: float,
    update_scale: float,
    eps: float = 1e-15,
) -> None:
    """One fused Muon update of ``param`` in place (see ``mi_muon_update_bf16``).

    ``momentum_buffer.lerp_(grad, 1 - beta)``; direction = ``grad.lerp(buffer, beta)`` if ``nesterov`` else the
    buffer; ``param = param_decay * param + update_scale * newton_schulz(direction)``.  The body of the
    parameter loop of the reference's ``OrthogonalizedOptimizer.step`` (orthogonalized_optimizer.py:185-210)
    for weight-decay methods that only scale the parameter.  All three tensors: GPU float32, same shape,
    contiguous, distinct storage.
    """
    if not (fused_supported(param) and grad.shape == param.shape and momentum_buffer.shape == param.shape):
        raise RuntimeError(f"fused_muon_update cannot take tensors of shape {tuple(param.shape)} / {tuple(grad.shape)}")
    for t, name in ((param, "param"), (grad, "grad"), (momentum_buffer, "momentum_buffer")):
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.device == param.device):
            raise RuntimeError(f"fused_muon_update: {name} must be a contiguous float32 tensor on {param.device}")
    if len(coefficients) < 1:
        raise ValueError("fused_muon_update needs at least one Newton-Schulz step")
    batch = param.shape[0] if param.dim() == 3 else 1
    rows, cols = param.shape[-2], param.shape[-1]
    lib = _hip.lib()
    flat = [float(v) for abc in coefficients for v in abc]
    abc = (ctypes.c_float * len(flat))(*flat)
    with torch.cuda.device(param.device):
        nbytes = lib.mi_newton_schulz_workspace_bytes(batch, rows, cols)
        ws = _launch.workspace(param.device, nbytes)
        rc = lib.mi_muon_update_bf16(
            _launch.ptr(param), _launch.ptr(grad), _launch.ptr(momentum_buffer), batch, rows, cols,
            float(beta), int(bool(nesterov)), float(param_decay), float(update_scale), abc, len(coefficients),
            float(eps), 0, _launch.ptr(ws), ws.numel(), _hip.current_stream_ptr(param.device),
        )  # fmt: skip
    _hip.check(rc)
