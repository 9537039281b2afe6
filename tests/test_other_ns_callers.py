"""Scion, Spel, PolarGrad and the spectral clipping utilities: the other callers of ``newton_schulz``.

CPU tests pin each against what its definition fixes (closed forms on the momentum buffer, singular values of the
result against a float64 SVD); the GPU tests check that ``use_syrk=True`` under "medium" precision (the HIP
kernels) stays within the bf16 tolerance of the float32 path.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn

from emerging_optimizers import orthogonalized_optimizers as oo
from emerging_optimizers import utils
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from oracle import ns_oracle as O



def _ns(x, steps=5, kind="quintic"):
    return torch.from_numpy(O.newton_schulz(x.numpy(), steps, kind)).float()


# ---------------------------------------------------------------- Scion
@pytest.mark.parametrize("shape", [(16, 24), (24, 16), (32, 32)])
def test_scion_step_is_a_frank_wolfe_step(shape):
    torch.manual_seed(0)
    p = nn.Parameter(torch.randn(shape))
    p0, g = p.detach().clone(), torch.randn(shape)
    p.grad = g.clone()
    lr, mom, radius = 0.1, 0.9, 2.0
    oo.Scion([p], lr=lr, momentum=mom, spectral_radius=radius, fp32_matmul_prec="highest").step()
    buf = (1 - mom) * g  # EMA from a zero buffer, no Nesterov
    want = (1 - lr) * p0 - lr * radius * (shape[0] / shape[1]) ** 0.5 * _ns(buf)
    torch.testing.assert_close(p.detach(), want, rtol=1e-4, atol=1e-5)


def test_scion_rejects_zero_steps():
    with pytest.raises(ValueError, match="num_ns_steps must be at least 1"):
        oo.Scion([nn.Parameter(torch.randn(4, 4))], num_ns_steps=0)


# ---------------------------------------------------------------- Spel
@pytest.mark.parametrize("shape", [(16, 24), (24, 16)])
def test_spel_reprojects_the_weight(shape):
    torch.manual_seed(1)
    p = nn.Parameter(torch.randn(shape))
    p0, g = p.detach().clone(), torch.randn(shape)
    p.grad = g.clone()
    lr, mom, wd = 0.05, 0.9, 0.1
    oo.Spel([p], lr=lr, momentum=mom, weight_decay=wd, fp32_matmul_prec="highest", coefficient_type="polar_express",
            num_ns_steps=8).step()
    inner = _ns((1 - mom) * g, 8, "polar_express")
    want = _ns((1 - lr * wd) * p0 - lr * inner, 8, "polar_express")
    torch.testing.assert_close(p.detach(), want, rtol=1e-4, atol=1e-5)
    sv = torch.linalg.svdvals(p.detach().double())
    assert float(sv.max()) < 1.2 and float(sv.min()) > 0.8  # the weight sits near the Stiefel manifold


# ---------------------------------------------------------------- PolarGrad
def test_polargrad_scales_by_the_nuclear_norm():
    torch.manual_seed(2)
    shape = (12, 20)
    p = nn.Parameter(torch.randn(shape))
    p0, g = p.detach().clone(), torch.randn(shape)
    p.grad = g.clone()
    lr, mom, wd, extra = 0.1, 0.5, 0.01, 0.2
    oo.PolarGrad([p], lr=lr, momentum=mom, weight_decay=wd, coefficient_type="polar_express", num_ns_steps=12,
                 extra_scale_factor=extra).step()
    buf = (1 - mom) * g
    u, s, vt = torch.linalg.svd(buf.double(), full_matrices=False)
    want = (1 - lr * wd) * p0.double() - lr * extra * float(s.sum()) * (u @ vt)  # exact polar factor x nuclear norm
    assert float((p.detach().double() - want).norm() / (want - p0.double()).norm()) < 2e-2
    # zero steps: the "orthogonalisation" is only the Frobenius normalisation, and the result is exact
    q = nn.Parameter(p0.clone())
    q.grad = g.clone()
    oo.PolarGrad([q], lr=lr, momentum=mom, weight_decay=0.0, num_ns_steps=0).step()
    nb = buf / buf.norm()
    torch.testing.assert_close(q.detach(), p0 - lr * nb * (nb * buf).sum(), rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError, match="num_ns_steps must be positive"):
        oo.PolarGrad([nn.Parameter(torch.randn(4, 4))], num_ns_steps=-1)


# ---------------------------------------------------------------- spectral clipping
def _svd_map(x, fn):
    u, s, vt = torch.linalg.svd(x.double(), full_matrices=False)
    return (u * fn(s)) @ vt


@pytest.mark.parametrize("dims", [(64, 32), (32, 64), (48, 48), (50, 100)])
@pytest.mark.parametrize("beta", [0.5, 1.0, 2.0])
def test_spectral_hardcap_caps_singular_values_and_keeps_singular_vectors(dims, beta):
    torch.manual_seed(3)
    x = torch.randn(dims) / dims[1] ** 0.5 * 1.5  # singular values spread around the caps
    with utils.fp32_matmul_precision("highest"):
        got = oo.spectral_hardcap(x, beta=beta)
    assert got.shape == x.shape
    want = _svd_map(x, lambda s: s.clamp(max=beta))
    assert float((got.double() - want).norm() / want.norm()) < 3e-2
    assert float(torch.linalg.svdvals(got.double()).max()) <= beta + 1e-1
    u0, _, v0 = torch.linalg.svd(x.double(), full_matrices=False)
    u1, _, v1 = torch.linalg.svd(got.double(), full_matrices=False)
    assert float(((u0 @ v0) - (u1 @ v1)).norm() / (u0 @ v0).norm()) <= 1e-4  # same polar factor


@pytest.mark.parametrize("dims", [(64, 32), (32, 64), (48, 48)])
@pytest.mark.parametrize("lo,hi", [(0.2, 0.8), (0.1, 20.0)])
def test_spectral_clip_clips_into_the_range(dims, lo, hi):
    torch.manual_seed(4)
    x = torch.randn(dims)
    with utils.fp32_matmul_precision("highest"):
        got = oo.spectral_clip(x, sigma_min=lo, sigma_max=hi)
    assert got.shape == x.shape
    sv = torch.linalg.svdvals(got.double())
    assert float(sv.min()) + 5e-1 >= lo and float(sv.max()) - 1e-1 <= hi  # the reference's own tolerances
    want = _svd_map(x, lambda s: s.clamp(min=lo, max=hi))
    assert float((got.double() - want).norm() / want.norm()) < 5e-2


def test_spectral_clipped_weight_decay_mixes_with_the_hardcap():
    torch.manual_seed(5)
    x = torch.randn(24, 40)
    with utils.fp32_matmul_precision("highest"):
        got = oo.spectral_clipped_weight_decay(x, beta=1.0, c=0.25)
        want = 0.75 * x + 0.25 * oo.spectral_hardcap(x, beta=1.0)
    torch.testing.assert_close(got, want)


# ---------------------------------------------------------------- GPU: the same callers on the HIP kernels
@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(512, 1024), (1024, 512)])
def test_callers_on_the_kernels_match_the_float32_path(gpu, shape):
    torch.manual_seed(6)
    w0 = torch.randn(shape) * 0.02
    g = torch.randn(shape) * 1e-3
    for cls, kw in ((oo.Scion, {}), (oo.Spel, {}), (oo.PolarGrad, {"fp32_matmul_prec": "medium"})):
        p, q = nn.Parameter(w0.clone().to(gpu)), nn.Parameter(w0.clone().to(gpu))
        p.grad, q.grad = g.clone().to(gpu), g.clone().to(gpu)
        fast = cls([p], lr=0.02, coefficient_type="simple", use_syrk=True, **kw)
        slow = cls([q], lr=0.02, coefficient_type="simple", **{**kw, "fp32_matmul_prec": "highest"})
        calls = []
        real = muon_utils.hip_kernels.fused_newton_schulz
        muon_utils.hip_kernels.fused_newton_schulz = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
        try:
            fast.step()
        finally:
            muon_utils.hip_kernels.fused_newton_schulz = real
        slow.step()
        assert len(calls) == (2 if cls is oo.Spel else 1), cls.__name__  # the kernels were used
        if cls is oo.Spel:  # the weight itself is the orthogonalised quantity
            rel = float((p.detach() - q.detach()).norm() / q.detach().norm())
        else:
            rel = float((p.detach() - q.detach()).norm() / (q.detach() - w0.to(gpu) * (1 - 0.02 * (1 if cls is oo.Scion else 0.01))).norm())
        assert rel <= 2e-2, (cls.__name__, rel)


@pytest.mark.gpu
def test_spectral_hardcap_on_the_kernels(gpu):
    torch.manual_seed(7)
    x = (torch.randn(512, 1024) / 32 * 1.5).to(gpu)
    with utils.fp32_matmul_precision("medium"):
        got = oo.spectral_hardcap(x, beta=1.0, use_syrk=True)
    want = _svd_map(x.cpu(), lambda s: s.clamp(max=1.0)).to(gpu)
    assert float((got.double() - want).norm() / want.norm()) < 3e-2


# ---------------------------------------------------------------- AdaptiveMuon
def _adaptive_by_hand(method, p0, g, *, lr, mom, wd, beta2, eps, nesterov, scale):
    """One step from zero state in float64 numpy, with the oracle's Newton-Schulz."""
    p = p0.double() * (1 - lr * wd)
    buf = (1 - mom) * g.double()
    m = (g.double() + mom * (buf - g.double())) if nesterov else buf
    o = _ns(m.float()).double()
    if method == "adamuon":
        v = (1 - beta2) * o**2
        u = o / (v.sqrt() + eps)
    elif method == "normuon":
        dim = -1 if o.shape[0] >= o.shape[1] else -2
        v = (1 - beta2) * (o**2).mean(dim=dim, keepdim=True)
        u = o / v.clamp_min(eps).sqrt()
        u = u * o.norm() / u.norm()
    else:
        v = (1 - beta2) * g.double().norm() ** 2
        u = o * m.norm() / (v.sqrt() + eps)
    return p - lr * scale * u, v


@pytest.mark.parametrize("method", ["adamuon", "normuon", "namo"])
@pytest.mark.parametrize("shape,nesterov", [((16, 24), False), ((24, 16), True)])
def test_adaptive_muon_step_by_hand(method, shape, nesterov):
    torch.manual_seed(8)
    p = nn.Parameter(torch.randn(shape))
    p0, g = p.detach().clone(), torch.randn(shape)
    p.grad = g.clone()
    kw = dict(lr=0.01, mom=0.9, wd=0.1, beta2=0.95, eps=1e-8, nesterov=nesterov)
    opt = oo.AdaptiveMuon([p], kw["lr"], kw["mom"], kw["wd"], nesterov=nesterov, moment2_method=method,
                          fp32_matmul_prec="highest", extra_scale_factor=0.5)
    opt.step()
    scale = 0.5 * oo.get_muon_scale_factor(*shape, mode="spectral")
    want, v = _adaptive_by_hand(method, p0, g, scale=scale, **kw)
    torch.testing.assert_close(p.detach().double(), want, rtol=2e-4, atol=2e-5)
    m2 = opt.state[p]["moment2_buffer"]
    want_shape = {"adamuon": shape, "namo": (1,),
                  "normuon": (shape[0], 1) if shape[0] >= shape[1] else (1, shape[1])}[method]
    assert tuple(m2.shape) == tuple(want_shape)
    torch.testing.assert_close(m2.double().reshape(-1), v.reshape(-1), rtol=2e-3, atol=1e-9)


@pytest.mark.parametrize("method", ["adamuon", "normuon", "namo"])
def test_adaptive_muon_scales_after_the_second_moment(method):
    torch.manual_seed(9)
    shape = (4, 16)
    w0, g = torch.randn(shape), torch.randn(shape)
    out = {}
    for mode in ("spectral", "shape_scaling"):
        p = nn.Parameter(w0.clone())
        p.grad = g.clone()
        opt = oo.AdaptiveMuon([p], 0.01, 0.0, 0.0, moment2_method=method, beta2=0.0, scale_mode=mode,
                              fp32_matmul_prec="highest")
        opt.step()
        out[mode] = (p.detach().clone(), opt.state[p]["moment2_buffer"].clone())
    assert torch.equal(out["spectral"][1], out["shape_scaling"][1])
    ratio = oo.get_muon_scale_factor(*shape, mode="spectral") / oo.get_muon_scale_factor(*shape, mode="shape_scaling")
    torch.testing.assert_close(w0 - out["spectral"][0], (w0 - out["shape_scaling"][0]) * ratio, rtol=1e-6, atol=1e-6)


def test_adaptive_muon_errors():
    with pytest.raises(ValueError, match='moment2_method="namo" is incompatible'):
        oo.AdaptiveMuon([nn.Parameter(torch.randn(4, 4))], 0.1, 0.9, 0.0, moment2_method="namo",
                        weight_decay_method="l2")
    with pytest.raises(ValueError, match="num_ns_steps must be at least 1"):
        oo.AdaptiveMuon([nn.Parameter(torch.randn(4, 4))], 0.1, 0.9, 0.0, num_ns_steps=0)
    for method in ("adamuon", "normuon", "namo"):
        p = nn.Parameter(torch.randn(8))
        p.grad = torch.randn(8)
        with pytest.raises(ValueError, match="only supports 2D"):
            oo.AdaptiveMuon([p], 0.1, 0.9, 0.0, moment2_method=method).step()
    p = nn.Parameter(torch.randn(4, 4))
    p.grad = torch.randn(4, 4)
    with pytest.raises(TypeError):
        oo.AdaptiveMuon([p], 0.1, 0.9, 0.0, moment2_method="nope").step()


# ---------------------------------------------------------------- MuonHyperball
@pytest.mark.parametrize("shape", [(16, 24), (32, 32)])
def test_muon_hyperball_keeps_the_norm_and_moves_along_the_update(shape):
    torch.manual_seed(10)
    radius, lr = 3.0, 0.05
    w = torch.randn(shape)
    w = w * radius / w.norm()
    p = nn.Parameter(w.clone())
    opt = oo.MuonHyperball([p], lr=lr, momentum=0.9, weight_decay=0.0, hyperball_radius=radius,
                           fp32_matmul_prec="highest")
    g = torch.randn(shape)
    p.grad = g.clone()
    opt.step()
    assert abs(float(p.detach().norm()) - radius) < 1e-5
    o = _ns(0.1 * g)
    moved = w - lr * radius * o / o.norm()
    torch.testing.assert_close(p.detach(), radius * moved / moved.norm(), rtol=1e-4, atol=1e-5)
    for _ in range(3):
        p.grad = torch.randn(shape)
        opt.step()
    assert abs(float(p.detach().norm()) - radius) < 1e-5


def test_muon_hyperball_errors():
    with pytest.raises(ValueError, match="non-zero norm"):
        oo.MuonHyperball([nn.Parameter(torch.zeros(4, 4))], lr=0.01, hyperball_radius=1.0)
    with pytest.raises(ValueError, match="hyperball_radius=1.0 was specified"):
        oo.MuonHyperball([nn.Parameter(torch.ones(4, 4))], lr=0.01, hyperball_radius=1.0)
    with pytest.raises(KeyError, match="weight_update_hook"):
        oo.MuonHyperball([nn.Parameter(torch.ones(4, 4) / 4)], lr=0.01, hyperball_radius=1.0,
                         weight_update_hook=object())
    from emerging_optimizers.weight_update_hooks import HyperballHook
    for bad in (dict(radius=float("inf")), dict(radius=1.0, eps=0.0), dict(radius=0.1, eps=0.25)):
        with pytest.raises(ValueError):
            HyperballHook(**bad)
    hook, tiny = HyperballHook(radius=2.0, eps=0.25), torch.full((2, 2), 0.01)
    hook.post_weight_update_inplace(tiny, None)
    assert float(tiny.abs().max()) == 0.0  # below eps: no direction to keep


@pytest.mark.gpu
@pytest.mark.parametrize("method", ["adamuon", "normuon", "namo"])
def test_adaptive_muon_on_the_kernels(gpu, method):
    torch.manual_seed(11)
    shape = (512, 1024)
    w0, g = torch.randn(shape) * 0.02, torch.randn(shape) * 1e-3
    res, m2 = [], []
    for kw in (dict(use_syrk=True, fp32_matmul_prec="medium"), dict(fp32_matmul_prec="highest")):
        p = nn.Parameter(w0.clone().to(gpu))
        p.grad = g.clone().to(gpu)
        opt = oo.AdaptiveMuon([p], 0.02, 0.9, 0.0, moment2_method=method, coefficient_type="simple", **kw)
        opt.step()
        res.append(p.detach() - w0.to(gpu))
        m2.append(opt.state[p]["moment2_buffer"].sqrt())
    assert float((m2[0] - m2[1]).norm() / m2[1].norm()) <= 2e-2
    if method == "adamuon":
        # from a zero second moment the first update is sign(O) / sqrt(1 - beta2): entries of O near zero may
        # flip under bf16 rounding, which is the method's own sensitivity and no property of the kernels
        assert float((res[0].sign() == res[1].sign()).float().mean()) >= 0.97
    else:
        rel = float((res[0] - res[1]).norm() / res[1].norm())
        assert rel <= 2e-2, (method, rel)


@pytest.mark.gpu
def test_muon_hyperball_on_the_kernels(gpu):
    torch.manual_seed(12)
    shape, radius = (1024, 512), 8.0
    w = torch.randn(shape)
    w = (w * radius / w.norm()).to(gpu)
    g = (torch.randn(shape) * 1e-3).to(gpu)
    res = []
    for kw in (dict(use_syrk=True, fp32_matmul_prec="medium"), dict(fp32_matmul_prec="highest")):
        p = nn.Parameter(w.clone())
        p.grad = g.clone()
        oo.MuonHyperball([p], lr=0.05, hyperball_radius=radius, coefficient_type="simple", **kw).step()
        assert abs(float(p.detach().norm()) - radius) < 1e-4
        res.append(p.detach() - w)
    assert float((res[0] - res[1]).norm() / res[1].norm()) <= 2e-2


# ---------------------------------------------------------------- same-shape parameters in one batched call
def _heads_model(device, n_heads=6):
    torch.manual_seed(13)
    ps = [nn.Parameter(torch.randn(128, 1024, device=device) * 0.02) for _ in range(n_heads)]
    ps += [nn.Parameter(torch.randn(256, 512, device=device) * 0.02), nn.Parameter(torch.randn(64, 64, device=device))]
    return ps


def _run_steps(ps, opt, n=2):
    g = torch.Generator().manual_seed(14)
    for _ in range(n):
        for p in ps:
            p.grad = (torch.randn(p.shape, generator=g) * 1e-3).to(p.device)
        opt.step()


@pytest.mark.parametrize("nesterov", [False, True])
def test_group_same_shape_equals_the_serial_loop(nesterov):
    a, b = _heads_model("cpu"), _heads_model("cpu")
    calls = []
    kw = dict(lr=0.05, nesterov=nesterov, weight_decay=0.01, fp32_matmul_prec="highest")
    grouped = oo.Muon(a, group_same_shape=True, **kw)
    real = grouped.scaled_orthogonalize_fn
    grouped.scaled_orthogonalize_fn = lambda t: (calls.append(tuple(t.shape)), real(t))[1]
    serial = oo.Muon(b, **kw)
    _run_steps(a, grouped)
    _run_steps(b, serial)
    assert sorted(calls[:3]) == [(6, 128, 1024), (64, 64), (256, 512)]  # one batched call for the six heads
    for p, q in zip(a, b):
        # (torch's batched and plain CPU matmuls differ in the last bits)
        torch.testing.assert_close(p.detach(), q.detach(), rtol=1e-5, atol=2e-6)
        assert torch.equal(grouped.state[p]["momentum_buffer"], serial.state[q]["momentum_buffer"])


def test_group_same_shape_leaves_overridden_orthogonalize_alone():
    class Split(oo.Muon):
        def orthogonalize(self, p, grad, **kwargs):
            return torch.cat([self.scaled_orthogonalize_fn(h) for h in grad.chunk(2, dim=0)], dim=0)

    ps = _heads_model("cpu", 2)
    opt = Split(ps, group_same_shape=True, fp32_matmul_prec="highest")
    assert opt._shapes_to_batch(opt.param_groups[0]) == set()
    _run_steps(ps, opt, 1)  # runs through the override, one parameter at a time


@pytest.mark.gpu
def test_group_same_shape_on_the_kernels(gpu):
    from emerging_optimizers.orthogonalized_optimizers import muon as muon_mod
    a, b = _heads_model(gpu), _heads_model(gpu)
    _run_steps(a, oo.Muon(a, lr=0.05, use_syrk=True, nesterov=True, group_same_shape=True))
    saved = muon_mod.FUSED_MUON_STEP
    muon_mod.FUSED_MUON_STEP = False  # the one-call update rounds the weight update differently
    try:
        _run_steps(b, oo.Muon(b, lr=0.05, use_syrk=True, nesterov=True))
    finally:
        muon_mod.FUSED_MUON_STEP = saved
    for p, q in zip(a[:6], b[:6]):
        assert torch.equal(p.detach(), q.detach())  # a batch entry is computed exactly as the matrix alone
    start = _heads_model(gpu)
    for p, q, p0 in zip(a[6:], b[6:], start[6:]):  # shapes that occur once keep the one-call update
        assert float((p.detach() - q.detach()).norm() / (q.detach() - p0.detach()).norm()) <= 1e-2
