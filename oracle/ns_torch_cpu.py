"""torch-on-CPU restatement of the reference's Newton-Schulz -- TEST/BENCH INFRASTRUCTURE, NOT PRODUCT CODE.

The reference has no separate CPU implementation: with ``device="cpu"`` it executes the torch operators
below (emerging_optimizers/orthogonalized_optimizers/muon_utils.py:216, 370-375).  This file restates that
operator sequence so that ``bench.py`` can time "the reference's CPU path" on the GPU box's host cores.
It is checked against ``ns_oracle.newton_schulz`` in ``tests/test_oracle.py``.
"""

import torch


def newton_schulz_cpu(x: torch.Tensor, coefficients, eps: float = 1e-15) -> torch.Tensor:
    """normalise -> per step { X @ X.mT ; addmm(A, A, A, alpha=c, beta=b) ; addmm(X, B, X, alpha=1, beta=a) }."""
    transpose = x.size(-2) > x.size(-1)
    if transpose:
        x = x.mT
    X = torch.nn.functional.normalize(x, p=2, dim=(-2, -1), eps=eps)
    for a, b, c in coefficients:
        A = X @ X.mT
        if c != 0.0:
            B = torch.addmm(A, A, A, alpha=c, beta=b)
            X = torch.addmm(X, B, X, alpha=1.0, beta=a)
        else:
            X = torch.addmm(X, A, X, alpha=b, beta=a)
    return X.mT if transpose else X
