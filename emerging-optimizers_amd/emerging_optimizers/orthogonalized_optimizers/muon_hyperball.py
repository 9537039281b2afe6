"""Muon on a sphere: update and weight are both rescaled to a fixed Frobenius norm.

Same constructor contract as the reference's ``MuonHyperball``
(orthogonalized_optimizers/muon_hyperball.py:29-95): every argument of :class:`Muon` (``use_syrk`` included),
plus the radius; a caller-supplied ``weight_update_hook`` is refused because the class installs its own.
"""

from __future__ import annotations

from typing import Any

import torch

from emerging_optimizers.orthogonalized_optimizers.muon import Muon
from emerging_optimizers.weight_update_hooks import HyperballHook


__all__ = ["MuonHyperball"]


class MuonHyperball(Muon[None]):
    """``W <- R * normalize(W - lr * R * normalize(update))`` with Muon's update.

    Args:
        *args: as for :class:`Muon`
        hyperball_radius: the Frobenius norm R every parameter already has (checked to rtol 1e-5)
        hyperball_eps: norms below this count as zero
        **kwargs: as for :class:`Muon`
    """

    def __init__(self, *args: Any, hyperball_radius: float, hyperball_eps: float = 1e-15, **kwargs: Any) -> None:
        if "weight_update_hook" in kwargs:
            raise KeyError(
                "MuonHyperball does not accept a 'weight_update_hook' argument; "
                "it manages its own HyperballHook internally."
            )
        super().__init__(*args, weight_update_hook=HyperballHook(hyperball_radius, hyperball_eps), **kwargs)
        with torch.no_grad():
            for group in self.param_groups:
                for p in group["params"]:
                    norm = float(torch.linalg.vector_norm(p, dtype=torch.float32))
                    if norm < hyperball_eps:
                        raise ValueError(
                            "MuonHyperball requires all parameters to have non-zero norm. "
                            "Found parameter with almost zero norm."
                        )
                    want = torch.tensor(hyperball_radius, dtype=torch.float32)
                    if not torch.isclose(torch.tensor(norm, dtype=torch.float32), want, atol=0, rtol=1e-5):
                        raise ValueError(
                            f"hyperball_radius={hyperball_radius} was specified but a parameter "
                            f"has Frobenius norm {norm}. Rescale your model parameters to the "
                            f"desired radius before constructing the optimizer."
                        )
