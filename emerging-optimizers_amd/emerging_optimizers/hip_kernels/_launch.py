"""Shared launch plumbing: tensors -> raw pointers/strides -> C ABI call on the current stream."""

from __future__ import annotations

import ctypes

import torch

from .. import _hip


def ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def require_gpu(t: torch.Tensor, who: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{who} runs on the GPU only; got a tensor on {t.device}")


def syrk_launch(
    mem_a: torch.Tensor,
    a_trans: bool,
    batch: int,
    n: int,
    k: int,
    c_mem: torch.Tensor | None,
    alpha: float,
    beta: float,
    d: torch.Tensor,
    skip_upper: bool,
) -> None:
    """``mem_a`` is the contiguous view of the operand: (B?, n, k) when not a_trans, else (B?, k, n)."""
    lib = _hip.lib()
    with torch.cuda.device(d.device):
        rc = lib.mi_syrk_bf16(
            ptr(mem_a), batch, n, k, n * k, mem_a.shape[-1], int(a_trans),
            ptr(c_mem), n * n, n, float(alpha), float(beta),
            ptr(d), n * n, n, int(bool(skip_upper)), _hip.current_stream_ptr(d.device),
        )  # fmt: skip
    _hip.check(rc)
