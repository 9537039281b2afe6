"""Shared test helpers (input generators for the benchmark configurations, comparison metrics)."""

import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")


def known_answer_cases():
    with open(GOLDEN) as f:
        doc = json.load(f)
    out = []
    for case in doc["cases"]:
        x = np.zeros((case["rows"], case["cols"]), dtype=np.float32)
        y = np.zeros((case["rows"], case["cols"]), dtype=np.float64)
        for r, c, v, e in zip(case["row_of"], case["col_of"], case["values"], case["expected"]):
            x[r, c] = v
            y[r, c] = e
        out.append((case, x, y))
    return out


def rel_fro(got, ref) -> float:
    got = torch.as_tensor(got, dtype=torch.float64)
    ref = torch.as_tensor(ref, dtype=torch.float64)
    return float((got - ref).norm() / ref.norm())


def through_bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(torch.float32)


def llama_grad(shape, seed, device="cpu"):
    """Gaussian 1e-3 entries with 1 % outliers at +-50 sigma (Llama-3-8B-shaped gradient stand-in)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * 1e-3
    mask = torch.rand(shape, generator=g) < 0.01
    sign = torch.where(torch.rand(shape, generator=g) < 0.5, -1.0, 1.0)
    x = torch.where(mask, sign * 50e-3, x)
    return x.to(device)


def ns_fp32_torch(x: torch.Tensor, coeffs, eps=1e-15) -> torch.Tensor:
    """float32 Newton-Schulz with torch ops on x's device ("highest" precision); reference for large shapes
    where the numpy oracle would take too long.  Checked against the oracle at small sizes in the tests."""
    prev = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("highest")
    try:
        tr = x.shape[-2] > x.shape[-1]
        X = x.mT if tr else x
        X = X / X.norm(dim=(-2, -1), keepdim=True).clamp_min(eps)
        for a, b, c in coeffs:
            A = X @ X.mT
            X = a * X + (b * A + c * (A @ A)) @ X if c != 0 else a * X + b * (A @ X)
        return X.mT if tr else X
    finally:
        torch.set_float32_matmul_precision(prev)
