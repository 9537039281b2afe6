"""Clipping of singular values through matrix sign functions, each computed by Newton-Schulz.

Same functions and arithmetic as the reference's ``spectral_clipping_utils``
(orthogonalized_optimizers/spectral_clipping_utils.py:24-98), after
https://leloykun.github.io/ponder/spectral-clipping/: ``clip(s, a, b) = ((a + b) + (a - s) sign(a - s)
- (b - s) sign(b - s)) / 2`` lifted to singular values, with ``msign`` from 8 "polar_express" steps.
``use_syrk`` is an addition (the reference fixes False); it is handed to ``newton_schulz``, which under matmul
precision "medium" runs float32 matrices on a gfx950 GPU on the kernels for either value.
"""

from __future__ import annotations

import torch

from emerging_optimizers.orthogonalized_optimizers.muon_utils import newton_schulz


__all__ = ["spectral_hardcap", "spectral_clip", "spectral_clipped_weight_decay"]


def _msign(x: torch.Tensor, use_syrk: bool) -> torch.Tensor:
    return newton_schulz(x, steps=8, coefficient_type="polar_express", use_syrk=use_syrk)


def spectral_clip(X: torch.Tensor, sigma_min: float = -1.0, sigma_max: float = 1.0, *, use_syrk: bool = False) -> torch.Tensor:
    """Clip the singular values of the 2-D ``X`` into ``[sigma_min, sigma_max]``, singular vectors unchanged."""
    tall = X.shape[0] > X.shape[1]
    W = X.T if tall else X
    O = _msign(W, use_syrk)
    eye = torch.eye(W.shape[0], device=W.device, dtype=W.dtype)
    out = (sigma_min + sigma_max) * O
    for bound, sign in ((sigma_min, 1.0), (sigma_max, -1.0)):
        gap_left = torch.addmm(bound * eye, O, W.T, beta=1.0, alpha=-1.0)  # bound I - O W^T  (m x m)
        gap = torch.add(bound * O, W, alpha=-1)                             # bound O - W      (m x n)
        out = torch.addmm(out, _msign(gap_left, use_syrk), gap, alpha=sign)
    out = out * 0.5
    return out.T if tall else out


def spectral_hardcap(X: torch.Tensor, beta: float = 1.0, *, use_syrk: bool = False) -> torch.Tensor:
    """Cap the singular values of the 2-D ``X`` at ``beta`` from above (``min(s, beta)``), singular vectors unchanged."""
    tall = X.shape[0] > X.shape[1]
    W = X.T if tall else X
    O = _msign(W, use_syrk)
    over = torch.add(beta * O, W, alpha=-1)  # beta O - W
    out = torch.add(beta * O, W)             # beta O + W
    out = torch.addmm(out, over, torch.mm(_msign(over, use_syrk).T, O), alpha=-1)
    out = out * 0.5
    return out.T if tall else out


def spectral_clipped_weight_decay(X: torch.Tensor, beta: float = 1.0, c: float = 0.5, *, use_syrk: bool = False) -> torch.Tensor:
    """Spectral counterpart of decoupled weight decay: ``(1 - c) X + c hardcap(X, beta)``."""
    return torch.add((1 - c) * X, spectral_hardcap(X, beta, use_syrk=use_syrk), alpha=c)
