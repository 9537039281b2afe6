"""GPU parity tests at the full size of the benchmark configurations that the smaller tests do not reach:
the stack of eight 4096 x 14336 expert gradients, and a whole ``Muon.step`` (momentum 0.95, Nesterov, weight
decay) on the Llama-3-8B attention and MLP shapes from a zero and from a warmed momentum buffer.

Reference at these sizes: the float32 Newton-Schulz / the float32 statement path of the optimizer, computed with
torch on the GPU under "highest" matmul precision (``ns_fp32_torch`` is itself checked against the numpy oracle at
a size both can do, ``test_gpu_torch_reference_is_trustworthy``).  Tolerance: relative Frobenius error <= 1e-2.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn as nn

from emerging_optimizers import utils
from emerging_optimizers.orthogonalized_optimizers import muon, muon_utils
from oracle import ns_oracle as O

from _helpers import llama_grad, ns_fp32_torch, rel_fro

pytestmark = pytest.mark.gpu
TOL_FP32 = 1e-2
SIMPLE5 = [(3.4445, -4.7750, 2.0315)] * 5


def test_stacked_experts_full_size(gpu):
    """8 experts x 4096 x 14336, Gaussian with per-expert scales log-uniform in [1e-4, 1e-2], 5 steps, one batched call."""
    g = torch.Generator().manual_seed(0)
    scales = torch.exp(torch.empty(8).uniform_(math.log(1e-4), math.log(1e-2), generator=g))
    dg = torch.Generator(device=gpu).manual_seed(0)
    x = torch.randn(8, 4096, 14336, device=gpu, generator=dg) * scales.to(gpu)[:, None, None]
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
    assert got.shape == x.shape and got.dtype == torch.float32
    errs = []
    for i in range(8):  # one expert at a time bounds the memory of the float32 reference
        ref = ns_fp32_torch(x[i], SIMPLE5)
        errs.append(rel_fro(got[i], ref))
        del ref
    print(f"\n  per-expert rel_fro vs fp32: {['%.2e' % e for e in errs]}")
    assert max(errs) <= TOL_FP32, errs
    # per-matrix normalisation: scaling every expert by a power of two changes nothing, bit for bit
    with utils.fp32_matmul_precision("medium"):
        got2 = muon_utils.newton_schulz(x * 4.0, steps=5, coefficient_type="simple", use_syrk=True)
    assert torch.equal(got, got2)
    # a batch entry is computed exactly as the matrix alone
    with utils.fp32_matmul_precision("medium"):
        alone = muon_utils.newton_schulz(x[3], steps=5, coefficient_type="simple", use_syrk=True)
    assert torch.equal(alone, got[3])


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 14336)])
def test_muon_step_full_size_zero_and_warmed_buffer(gpu, shape):
    """Llama-like gradients (N(0, 1e-3^2), 1 % entries at 50 sigma); momentum 0.95 with Nesterov and decoupled weight
    decay 0.01.  Step 1 starts from a zero buffer (buf = 0.05 g, direction = 0.05 g + 0.95 buf), step 4 runs on a
    buffer warmed by three seeded gradients.  The kernel path (one fused library call per step) against the same
    optimizer run statement by statement in float32."""
    lr, wd = 0.02, 0.01
    w0 = torch.randn(shape, generator=torch.Generator().manual_seed(1)) * 0.02
    p, q = nn.Parameter(w0.clone().to(gpu)), nn.Parameter(w0.clone().to(gpu))
    kw = dict(lr=lr, momentum=0.95, nesterov=True, weight_decay=wd, coefficient_type="simple")
    fast = muon.Muon([p], use_syrk=True, **kw)
    slow = muon.Muon([q], fp32_matmul_prec="highest", **kw)
    assert fast.use_syrk
    for step in range(1, 5):
        g = llama_grad(shape, seed=300 + step).to(gpu)
        p.grad, q.grad = g.clone(), g.clone()
        before_p, before_q = p.detach().clone(), q.detach().clone()
        fast.step()
        slow.step()
        torch.testing.assert_close(fast.state[p]["momentum_buffer"], slow.state[q]["momentum_buffer"], rtol=2e-6, atol=5e-9)
        if step in (1, 4):
            upd_fast = p.detach() - before_p * (1 - lr * wd)
            upd_slow = q.detach() - before_q * (1 - lr * wd)
            err = float((upd_fast - upd_slow).norm() / upd_slow.norm())
            # update = -lr sqrt(max(shape)) NS(direction): singular values near 1 make its RMS close to lr
            rms = float(upd_fast.pow(2).mean().sqrt()) / lr
            print(f"\n  {shape} step {step}: update rel_fro vs float32 statements = {err:.3e}, RMS / lr = {rms:.3f}")
            assert err <= TOL_FP32
            assert 0.6 < rms < 1.2
    assert torch.isfinite(p).all()


@pytest.mark.parametrize("shape", [(4096, 14336), (14336, 4096), (4096, 4096)])
def test_default_muon_runs_on_the_kernels_full_size(gpu, monkeypatch, shape):
    """`Muon(params)` with every argument at the reference's default (use_syrk=False, "quintic", no Nesterov, matmul
    precision "medium"): each step is one fused library call, and the update is within 1e-2 of the same optimizer
    run statement by statement in float32."""
    from emerging_optimizers import hip_kernels

    calls = []
    real = hip_kernels.fused_muon_update
    monkeypatch.setattr(hip_kernels, "fused_muon_update", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    w0 = torch.randn(shape, generator=torch.Generator().manual_seed(2)) * 0.02
    p, q = nn.Parameter(w0.clone().to(gpu)), nn.Parameter(w0.clone().to(gpu))
    fast = muon.Muon([p])
    slow = muon.Muon([q], fp32_matmul_prec="highest")
    assert not fast.use_syrk
    lr, wd = fast.param_groups[0]["lr"], fast.param_groups[0]["weight_decay"]
    for step in range(1, 3):
        g = llama_grad(shape, seed=400 + step).to(gpu)
        p.grad, q.grad = g.clone(), g.clone()
        before_p, before_q = p.detach().clone(), q.detach().clone()
        fast.step()
        slow.step()
        assert len(calls) == step
        # (the parameter moves by lr = 3e-4 times an O(1) update: the difference of two float32 values of size 0.02
        # carries their rounding, 1e-9 against an update of 3e-4 -- far below the tolerance)
        upd_fast = p.detach() - before_p * (1 - lr * wd)
        upd_slow = q.detach() - before_q * (1 - lr * wd)
        err = float((upd_fast - upd_slow).norm() / upd_slow.norm())
        print(f"\n  default Muon {shape} step {step}: update rel_fro vs float32 statements = {err:.3e}")
        assert err <= TOL_FP32
    torch.testing.assert_close(fast.state[p]["momentum_buffer"], slow.state[q]["momentum_buffer"], rtol=2e-6, atol=5e-9)


def test_grouped_muon_step_against_the_oracle(gpu):
    """Same-shape parameters orthogonalised in one batched call (group_same_shape=True), on the kernels, against the
    numpy oracle's optimizer step with its float32 Newton-Schulz."""
    torch.manual_seed(13)
    heads = [nn.Parameter((torch.randn(128, 1024) * 0.02).to(gpu)) for _ in range(6)]
    start = [p.detach().cpu().numpy().copy() for p in heads]
    lr, wd, beta = 0.05, 0.01, 0.95
    opt = muon.Muon(heads, lr=lr, momentum=beta, nesterov=True, weight_decay=wd, coefficient_type="quintic", use_syrk=True,
                    group_same_shape=True)
    calls = []
    real = opt.scaled_orthogonalize_fn
    opt.scaled_orthogonalize_fn = lambda t: (calls.append(tuple(t.shape)), real(t))[1]
    want = [s.copy() for s in start]
    bufs = [np.zeros_like(s) for s in start]
    gen = torch.Generator().manual_seed(14)
    for _ in range(2):
        grads = [torch.randn(128, 1024, generator=gen) * 1e-3 for _ in heads]
        for p, g in zip(heads, grads):
            p.grad = g.to(gpu)
        opt.step()
        for i, g in enumerate(grads):
            want[i], bufs[i] = O.optimizer_step(
                want[i], g.numpy(), bufs[i], lr=lr, momentum=beta, weight_decay=wd, weight_decay_method="decoupled", nesterov=True,
                orthogonalize=lambda d: O.muon_orthogonalize(d, steps=5, coefficient_type="quintic", scale_mode="spectral",
                                                             precision="highest"))
    assert calls == [(6, 128, 1024)] * 2  # one batched orthogonalisation per step
    for p, w, s, b in zip(heads, want, start, bufs):
        got = p.detach().cpu().numpy()
        assert np.linalg.norm(got - w) / np.linalg.norm(w - s) <= TOL_FP32
        np.testing.assert_allclose(opt.state[p]["momentum_buffer"].cpu().numpy(), b, rtol=1e-5, atol=1e-9)


# ---------------------------------------------------------------- hard spectra at the sizes where steps are grouped
def _hard_matrix(kind, m, n, gen, dev):
    """Inputs whose spectra are nothing like a Gaussian matrix's: power laws, low rank plus noise, heavy tails."""
    if kind in ("flat power law", "steep power law"):
        u, _ = torch.linalg.qr(torch.randn(m, m, device=dev, generator=gen))
        v, _ = torch.linalg.qr(torch.randn(n, m, device=dev, generator=gen))
        k = torch.arange(1, m + 1, dtype=torch.float32, device=dev)
        return (u * k ** (-0.5 if kind.startswith("flat") else -1.0)) @ v.mT
    if kind == "rank 64 + 10% noise":
        low = torch.randn(m, 64, device=dev, generator=gen) @ torch.randn(64, n, device=dev, generator=gen) / 8
        return low + 0.1 * torch.randn(m, n, device=dev, generator=gen)
    if kind == "student-t(3) entries":
        z = torch.randn(m, n, device=dev, generator=gen)
        chi2 = sum(torch.randn(m, n, device=dev, generator=gen) ** 2 for _ in range(3))
        return z / (chi2 / 3).sqrt()
    raise ValueError(kind)


HARD_KINDS = ["flat power law", "steep power law", "rank 64 + 10% noise", "student-t(3) entries"]


@pytest.mark.parametrize("kind", ["simple", "quintic"])
@pytest.mark.parametrize("shape", [(4096, 14336), (8, 1792, 4096)])
def test_grouped_steps_on_hard_spectra_at_full_size(gpu, mi_option, shape, kind):
    """The default grouping (3 + 2 for five quintic steps on wide matrices) against single steps, at the sizes where
    the rule switches grouping on and on inputs with power-law, low-rank and heavy-tailed spectra: such inputs are far
    from float32 under any bf16 schedule, the reference's included; what must hold is that grouping does not add to
    that.  Reference: the same iteration in float64 on the GPU."""
    gen = torch.Generator(device=gpu).manual_seed(17)
    coeffs = O.expand_coefficients(5, kind)
    m, n = shape[-2:]
    if len(shape) == 2:
        cases = [(k, _hard_matrix(k, m, n, gen, gpu)) for k in HARD_KINDS]
    else:  # a stack whose entries cycle through the four kinds at different scales
        stack = torch.stack([_hard_matrix(HARD_KINDS[i % 4], m, n, gen, gpu) * 10.0 ** (-i) for i in range(shape[0])])
        cases = [("stack of " + ", ".join(HARD_KINDS), stack)]
    for name, x in cases:
        want = ns_fp32_torch(x.double(), coeffs)
        err = {}
        for label, option in (("auto", -1), ("single", 0)):
            mi_option("ns_pairs", option)
            with utils.fp32_matmul_precision("medium"):
                got = muon_utils.newton_schulz(x, steps=5, coefficient_type=kind)
            d = (got.double() - want).flatten(-2).norm(dim=-1) / want.flatten(-2).norm(dim=-1)
            err[label] = d.flatten().tolist()
            del got
        print(f"\n  {shape} {kind} {name}: auto {['%.2e' % e for e in err['auto']]} single {['%.2e' % e for e in err['single']]}")
        for a, s in zip(err["auto"], err["single"]):
            assert a <= 1.15 * s + 5e-4, (name, kind, err)
        del want
