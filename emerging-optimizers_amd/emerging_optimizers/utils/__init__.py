"""Small helpers used on the orthogonalisation path."""

from __future__ import annotations

import contextlib
from typing import Iterator, Literal

import torch


__all__ = ["fp32_matmul_precision", "FP32MatmulPrecT"]

FP32MatmulPrecT = Literal["highest", "high", "medium"]


@contextlib.contextmanager
def fp32_matmul_precision(precision: FP32MatmulPrecT = "highest") -> Iterator[None]:
    """Temporarily set ``torch.set_float32_matmul_precision`` (reference: utils/__init__.py:28-40).

    On this path the setting is more than a hint: ``"medium"`` is what switches ``newton_schulz`` to its
    bf16 kernels (muon_utils.py:245 of the reference).
    """
    saved = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision(precision)
    try:
        yield
    finally:
        torch.set_float32_matmul_precision(saved)
