"""Host side of the package on CPU tensors, checked against the numpy oracle and the expectations the
reference's own tests state (tests/test_muon_utils.py, tests/test_orthogonalized_optimizer.py there)."""

import math

import numpy as np
import pytest
import torch
import torch.nn as nn

from emerging_optimizers import utils
from emerging_optimizers.orthogonalized_optimizers import muon, muon_utils
from emerging_optimizers.orthogonalized_optimizers.orthogonalized_optimizer import OrthogonalizedOptimizer
from oracle import ns_oracle as O

from _helpers import known_answer_cases


@pytest.fixture(autouse=True)
def _highest():
    torch.set_float32_matmul_precision("highest")


def test_tables_match_oracle():
    assert muon_utils._COEFFICIENT_SETS == O.COEFFICIENT_SETS


# newton_schulz on CPU vs oracle; tolerances are the reference's (test_muon_utils.py:109-122, 269-320 there)
@pytest.mark.parametrize("shape", [(128, 128), (128, 64), (64, 128)])
@pytest.mark.parametrize("kind,steps,atol", [("quintic", 5, 1e-6), ("cubic5", 5, 1e-6), ("cans", 5, 1e-5),
                                             ("polar_express", 9, 2e-6), ("deepseekv4", 10, 2e-6), ("cans", 9, 2e-6)])
def test_newton_schulz_cpu_matches_oracle(shape, kind, steps, atol):
    x = torch.randn(*shape)
    got = muon_utils.newton_schulz(x, steps=steps, coefficient_type=kind)
    want = O.newton_schulz(x.numpy(), steps, kind)
    assert got.dtype == torch.float32 and got.shape == x.shape
    np.testing.assert_allclose(got.numpy(), want, atol=atol, rtol=1e-6)


def test_newton_schulz_known_answers():
    for case, x, want in known_answer_cases():
        got = muon_utils.newton_schulz(torch.from_numpy(x), steps=case["steps"], coefficient_type=case["coefficient_type"])
        np.testing.assert_allclose(got.numpy(), want, atol=2e-6, rtol=1e-5)


def test_newton_schulz_close_to_svd():
    x = torch.randn(256, 128)
    out = muon_utils.newton_schulz(x, steps=5, coefficient_type="quintic")
    u, _, vt = torch.linalg.svd(x, full_matrices=False)
    torch.testing.assert_close(out, u @ vt, atol=1e-1, rtol=1e-7)


def test_custom_coefficients():
    x = 2 ** torch.randint(-10, -5, (65, 33)).float()
    sets = [(3, 5, 7), (11, 13, 17)]
    got = muon_utils.newton_schulz(x, steps=2, coefficient_type="custom", custom_coefficient_sets=sets)
    want = O.newton_schulz(x.numpy(), 2, "custom", custom_coefficient_sets=sets, compute_dtype=np.float64)
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-5, atol=0)


def test_underflowed_norm_in_fp64():
    x = torch.randn(256, 256) * 1e-30
    assert torch.linalg.vector_norm(x) == 0
    norm_ref = torch.linalg.vector_norm(x, dtype=torch.double)
    out = muon_utils.newton_schulz(x, steps=0, normalize_in_double=True)
    torch.testing.assert_close(x / norm_ref, out, atol=0, rtol=1e-6)


@pytest.mark.parametrize("kind", ["quintic", "cubic5"])
@pytest.mark.parametrize("shape", [(2, 64, 64), (4, 32, 64), (3, 64, 32)])
def test_3d_equals_per_slice(shape, kind):
    x = torch.randint(-3, 4, shape).float()
    out = muon_utils.newton_schulz(x, steps=5, coefficient_type=kind)
    per = torch.stack([muon_utils.newton_schulz(x[i], steps=5, coefficient_type=kind) for i in range(shape[0])])
    torch.testing.assert_close(out, per, atol=1e-6, rtol=0)


def test_medium_precision_cpu_follows_bf16_schedule():
    x = torch.randn(64, 96)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple")
    want = O.newton_schulz(x.numpy(), 5, "simple", precision="medium")
    # same rounding points, different summation order inside the matmuls: a few bf16 ulps on few entries
    assert np.linalg.norm(got.numpy() - want) / np.linalg.norm(want) < 3e-3


def test_polar_express_beats_quintic_on_ill_conditioned_input():
    u, _ = torch.linalg.qr(torch.randn(128, 128))
    v, _ = torch.linalg.qr(torch.randn(128, 128))
    x = u @ torch.diag(torch.logspace(6, -6, 128)) @ v.T
    ref = u @ v.T
    for kind in ("polar_express", "deepseekv4"):
        better = torch.linalg.vector_norm(muon_utils.newton_schulz(x, steps=10, coefficient_type=kind) - ref)
        base = torch.linalg.vector_norm(muon_utils.newton_schulz(x, steps=5, coefficient_type="quintic") - ref)
        assert better < base


def test_error_paths():
    for shape in [(10,), (2, 3, 4, 5)]:
        with pytest.raises(TypeError, match="must be 2d or 3d"):
            muon_utils.newton_schulz(torch.randn(*shape), steps=5)
    with pytest.raises(TypeError, match="float32.*float64"):
        muon_utils.newton_schulz(torch.randn(5, 7, dtype=torch.float64), steps=5)
    x = torch.randn(5, 7)
    with pytest.raises(ValueError, match="custom_coefficient_sets must be provided"):
        muon_utils.newton_schulz(x, steps=5, coefficient_type="custom")
    with pytest.raises(ValueError, match="Invalid coefficient type.*nonexistent"):
        muon_utils.newton_schulz(x, steps=5, coefficient_type="nonexistent")
    for steps in (1, 4, 6):
        with pytest.raises(ValueError, match="cubic5.*fixed.*5-step schedule.*steps=5"):
            muon_utils.newton_schulz(x, steps=steps, coefficient_type="cubic5")
    with pytest.raises(ValueError, match="must be non-empty"):
        list(muon_utils.get_coefficient_iterator(5, []))
    with pytest.raises(ValueError, match="Invalid mode.*invalid"):
        list(muon_utils.get_coefficient_iterator(5, [(1.0, 2.0, 3.0)], mode="invalid"))
    with pytest.raises(ValueError, match="Invalid partition_dim.*2"):
        muon_utils.newton_schulz_tp(x, steps=5, coefficient_type="quintic", tp_group=None, partition_dim=2, tp_mode="distributed")
    with pytest.raises(ValueError, match="Invalid tp_mode.*invalid"):
        muon_utils.newton_schulz_tp(x, steps=5, coefficient_type="quintic", tp_group=None, partition_dim=0, tp_mode="invalid")
    torch.testing.assert_close(
        muon_utils.newton_schulz_tp(x, steps=5, coefficient_type="quintic", tp_group=None),
        muon_utils.newton_schulz(x, steps=5, coefficient_type="quintic"),
    )


def test_input_not_mutated_and_iterator_values():
    x = torch.randn(16, 24)
    keep = x.clone()
    muon_utils.newton_schulz(x, steps=3)
    assert torch.equal(x, keep)
    sets = muon_utils._COEFFICIENT_SETS["quintic"]
    assert list(muon_utils.get_coefficient_iterator(7, sets)) == [sets[i % 5] for i in range(7)]
    assert list(muon_utils.get_coefficient_iterator(7, sets, "repeat_last")) == [sets[min(i, 4)] for i in range(7)]


@pytest.mark.parametrize("shape", [(4, 4), (4, 8), (8, 4), (2, 4, 8), (2, 8, 4)])
def test_use_syrk_falls_back_for_unaligned_shapes(shape, monkeypatch):
    """Shapes that are not multiples of 8 must go through the library-GEMM step exactly once per step and
    never reach the SYRK step, even with use_syrk=True under "medium" (test_muon_utils.py:350-403 there)."""
    calls = {"n": 0}
    name = "newton_schulz_step" if len(shape) == 2 else "batched_newton_schulz_step"
    original = getattr(muon_utils, name)

    def counting(X, a, b, c, tp_group=None):
        calls["n"] += 1
        return original(X, a, b, c, tp_group=tp_group)

    def forbidden(X, a, b, c, tp_group=None):
        raise AssertionError("SYRK step must not run for a shape that is not a multiple of 8")

    monkeypatch.setattr(muon_utils, name, counting)
    monkeypatch.setattr(muon_utils, "newton_schulz_step_tsyrk", forbidden)
    monkeypatch.setattr(muon_utils, "batched_newton_schulz_step_tsyrk", forbidden)
    with utils.fp32_matmul_precision("medium"):
        muon_utils.newton_schulz(torch.randn(shape), steps=1, coefficient_type="simple", use_syrk=True)
    assert calls["n"] == 1


def test_step_functions_cpu():
    x = torch.randint(-3, 4, (4, 16, 32)).float()
    x = torch.nn.functional.normalize(x, p=2, dim=(-2, -1), eps=1e-7)
    a, b, c = 0.5, 1, 0.25
    batched = muon_utils.batched_newton_schulz_step(x, a, b, c)
    per = torch.stack([muon_utils.newton_schulz_step(x[i], a, b, c) for i in range(4)])
    torch.testing.assert_close(batched, per, atol=1e-8, rtol=0)
    np.testing.assert_allclose(batched.numpy(), O.newton_schulz_step(x.numpy(), a, b, c), atol=1e-6)
    cubic = muon_utils.batched_newton_schulz_step(x, 2.0, -1.5, 0.0)
    torch.testing.assert_close(cubic, 2.0 * x - 1.5 * ((x @ x.mT) @ x), atol=1e-6, rtol=1e-7)


def test_fp32_matmul_precision_context():
    torch.set_float32_matmul_precision("highest")
    with utils.fp32_matmul_precision("medium"):
        assert torch.get_float32_matmul_precision() == "medium"
        with pytest.raises(RuntimeError):
            with utils.fp32_matmul_precision("high"):
                raise RuntimeError("boom")
        assert torch.get_float32_matmul_precision() == "medium"
    assert torch.get_float32_matmul_precision() == "highest"


# ---------------------------------------------------------------- optimizer classes
@pytest.mark.parametrize("shape", [(5, 7), (33, 65), (127, 257)])
def test_core_matches_sgd(shape):
    p = nn.Parameter(torch.randint(-5, 5, shape).float())
    q = nn.Parameter(p.detach().clone())
    p.grad = torch.randint_like(p, -5, 5)
    q.grad = p.grad.clone()
    opt = OrthogonalizedOptimizer([p], lr=2, momentum=0, nesterov=False, weight_decay=0.5,
                                  weight_decay_method="decoupled", fp32_matmul_prec="highest")
    sgd = torch.optim.SGD([q], lr=2, momentum=0, nesterov=False, weight_decay=0.5)
    before, grad = p.detach().clone().numpy(), p.grad.clone().numpy()
    opt.step()
    sgd.step()
    assert torch.equal(p.data, q.data)
    want, _ = O.optimizer_step(before, grad, np.zeros_like(before), lr=2, momentum=0, weight_decay=0.5)
    np.testing.assert_array_equal(p.detach().numpy(), want)


@pytest.mark.parametrize("shape", [(5, 7), (33, 65)])
def test_core_matches_sgd_with_momentum(shape):
    p = nn.Parameter(torch.randint(-5, 5, shape).float())
    q = nn.Parameter(p.detach().clone())
    opt = OrthogonalizedOptimizer([p], lr=2.0, momentum=0.5, nesterov=False, weight_decay=0.0,
                                  weight_decay_method="l2", fp32_matmul_prec="highest")
    sgd = torch.optim.SGD([q], lr=1.0, momentum=0.5, nesterov=False, weight_decay=0.0)
    for _ in range(5):
        p.grad = torch.randint_like(p, -5, 5)
        q.grad = p.grad.clone()
        opt.step()
        sgd.step()
    assert torch.equal(p.data, q.data)


@pytest.mark.parametrize("method", ["decoupled", "independent", "l2", "palm"])
@pytest.mark.parametrize("nesterov", [True, False])
def test_step_matches_oracle_all_flavours(method, nesterov):
    p = nn.Parameter(torch.randn(9, 11))
    opt = OrthogonalizedOptimizer([p], lr=0.3, momentum=0.9, nesterov=nesterov, weight_decay=0.1,
                                  weight_decay_method=method, fp32_matmul_prec="highest")
    pn, buf = p.detach().numpy().copy(), np.zeros((9, 11), np.float32)
    for _ in range(3):
        g = torch.randn(9, 11)
        p.grad = g.clone()
        opt.step()
        pn, buf = O.optimizer_step(pn, g.numpy(), buf, lr=0.3, momentum=0.9, weight_decay=0.1,
                                   weight_decay_method=method, nesterov=nesterov)
    np.testing.assert_allclose(p.detach().numpy(), pn, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("skip", [False, True])
def test_init_group(skip):
    a, b = nn.Parameter(torch.randn(5, 7)), nn.Parameter(torch.randn(5, 7))
    a.grad = torch.randn_like(a)
    opt = OrthogonalizedOptimizer([a, b], lr=1.0, momentum=0.0, nesterov=False, weight_decay=0.0,
                                  weight_decay_method="l2", fp32_matmul_prec="highest")
    opt._init_group(opt.param_groups[0], skip_non_grad_params=skip)
    assert opt.state[a]["momentum_buffer"].shape == a.shape
    assert ("momentum_buffer" in opt.state[b]) == (not skip)


def test_custom_orthogonalize_fn_and_errors():
    p = torch.zeros((6, 7))
    p.grad = torch.arange(1, 7).float()[:, None].expand(6, 7).contiguous()

    def fn(x):
        groups = [x[i::3] for i in range(3)]
        return torch.cat([torch.full_like(g, g.max()) for g in groups], dim=0)

    opt = OrthogonalizedOptimizer([p], lr=-1, momentum=0, nesterov=False, weight_decay=0.0,
                                  weight_decay_method="l2", fp32_matmul_prec="highest", scaled_orthogonalize_fn=fn)
    opt.step()
    assert torch.equal(p, fn(p.grad))
    q = nn.Parameter(torch.randn(8))
    q.grad = torch.randn(8)
    bad = OrthogonalizedOptimizer([q], lr=1.0, momentum=0.0, weight_decay=0.0, nesterov=False,
                                  weight_decay_method="l2", fp32_matmul_prec="highest")
    with pytest.raises(ValueError, match="Only 2D"):
        bad.step()
    with pytest.raises(ValueError, match="closure is not supported"):
        bad.step(lambda: 0.0)


@pytest.mark.parametrize("shape", [(5, 7), (33, 65), (127, 257)])
@pytest.mark.parametrize("method", ["decoupled", "independent", "l2"])
@pytest.mark.parametrize("nesterov", [True, False])
def test_muon_smoke(shape, method, nesterov):
    p = nn.Parameter(torch.randint(-5, 5, shape).float())
    p.grad = torch.randint_like(p, -5, 5)
    muon.Muon([p], weight_decay_method=method, nesterov=nesterov).step()
    assert torch.isfinite(p).all()


def test_muon_update_matches_oracle():
    p = nn.Parameter(torch.randn(24, 40))
    g = torch.randn(24, 40)
    p.grad = g.clone()
    before = p.detach().numpy().copy()
    opt = muon.Muon([p], lr=0.02, momentum=0.95, nesterov=True, weight_decay=0.0, fp32_matmul_prec="highest",
                    coefficient_type="simple")
    opt.step()
    want, _ = O.optimizer_step(before, g.numpy(), np.zeros_like(before), lr=0.02, momentum=0.95, weight_decay=0.0,
                               nesterov=True, orthogonalize=lambda m: O.muon_orthogonalize(m, coefficient_type="simple", precision="highest"))
    np.testing.assert_allclose(p.detach().numpy(), want, atol=2e-5)


def test_muon_properties_and_validation():
    opt = muon.Muon([nn.Parameter(torch.randn(5, 7))])
    assert (opt.num_ns_steps, opt.coefficient_type, opt.scale_mode, opt.extra_scale_factor, opt.use_syrk) == (5, "quintic", "spectral", 1.0, False)
    for name in ("num_ns_steps", "coefficient_type", "scale_mode", "extra_scale_factor", "use_syrk"):
        with pytest.raises(AttributeError, match=f"Cannot set `{name}`"):
            setattr(opt, name, getattr(opt, name))
    with pytest.raises(ValueError, match="num_ns_steps must be at least 1"):
        muon.Muon([nn.Parameter(torch.randn(5, 7))], num_ns_steps=0)
    with pytest.raises(ValueError, match="Invalid mode.*invalid_mode"):
        muon.get_muon_scale_factor(10, 10, "invalid_mode")
    for o, i in [(512, 512), (512, 256), (97, 37), (37, 97)]:
        assert muon.get_muon_scale_factor(o, i, "shape_scaling") == math.sqrt(max(1, o / i))
        assert muon.get_muon_scale_factor(o, i, "spectral") == math.sqrt(max(o, i))
        assert muon.get_muon_scale_factor(o, i, "unit_rms_norm") == math.sqrt(o / i)


def test_muon_independent_weight_decay():
    p = nn.Parameter(torch.randint(-5, 5, (32, 32)).float())
    p.grad = torch.randint_like(p, -5, 5)
    want = 0.75 * p.data
    muon.Muon([p], lr=0.0, weight_decay=0.25, weight_decay_method="independent", momentum=0.0).step()
    assert torch.equal(p.data, want)


def test_muon_use_syrk_without_gpu_downgrades():
    if torch.cuda.is_available():
        pytest.skip("CPU-only behaviour")
    assert muon.Muon([nn.Parameter(torch.randn(8, 8))], use_syrk=True).use_syrk is False


def test_per_head_equivalence_cpu():
    """3-D stacked heads, and a list of independent 2-D heads, give the same update (per-head Muon)."""
    heads, d, n = 4, 16, 64
    g = torch.randn(heads * d, n)
    fn = muon.Muon([nn.Parameter(torch.zeros(d, n))], fp32_matmul_prec="highest").scaled_orthogonalize_fn
    stacked = fn(g.view(heads, d, n)).reshape(heads * d, n)
    separate = torch.cat([fn(g[i * d:(i + 1) * d]) for i in range(heads)])
    torch.testing.assert_close(stacked, separate, atol=1e-6, rtol=0)
