"""Pins the CPU oracle (oracle/ns_oracle.py) with checks that do not reuse its own formulas:
closed forms, brute force on tiny inputs, scalar known answers, invariants.  CPU only."""

import math

import numpy as np
import pytest

from oracle import ns_oracle as O

from _helpers import known_answer_cases


# ---------------------------------------------------------------- coefficient tables / iterator
def test_table_fixed_points():
    a, b, c = O.COEFFICIENT_SETS["simple"][0]
    assert a + b + c == pytest.approx(0.7010, abs=1e-12)
    a, b, c = O.COEFFICIENT_SETS["polar_express"][-1]
    assert (a, b, c) == (15 / 8, -10 / 8, 3 / 8)
    assert a + b + c == 1.0 and a + 3 * b + 5 * c == 0.0  # p(1) = 1, p'(1) = 0
    a, b, c = O.COEFFICIENT_SETS["deepseekv4"][-1]
    assert a + b + c == 1.0
    assert [len(O.COEFFICIENT_SETS[k]) for k in ("simple", "quintic", "polar_express", "cans", "aol", "deepseekv4", "cubic5")] == [1, 5, 8, 5, 4, 10, 5]
    assert all(c == 0.0 for _, _, c in O.COEFFICIENT_SETS["cubic5"])
    assert O.COEFFICIENT_SETS["deepseekv4"][:8] == [O.COEFFICIENT_SETS["simple"][0]] * 8


@pytest.mark.parametrize("steps", [0, 1, 3, 7])
def test_iterator_closed_form(steps):
    sets = [(1.0, 2.0, 3.0), (4.0, 5.0, 6.0), (7.0, 8.0, 9.0)]
    assert list(O.coefficient_iterator(steps, sets, "cycle")) == [sets[i % 3] for i in range(steps)]
    assert list(O.coefficient_iterator(steps, sets, "repeat_last")) == [sets[min(i, 2)] for i in range(steps)]


def test_iterator_errors():
    with pytest.raises(ValueError, match="must be non-empty"):
        list(O.coefficient_iterator(5, []))
    with pytest.raises(ValueError, match="Invalid mode.*invalid"):
        list(O.coefficient_iterator(5, [(1.0, 2.0, 3.0)], mode="invalid"))
    with pytest.raises(ValueError, match="cubic5.*fixed.*5-step schedule.*steps=5"):
        O.expand_coefficients(4, "cubic5")
    with pytest.raises(ValueError, match="custom_coefficient_sets must be provided"):
        O.expand_coefficients(4, "custom")
    with pytest.raises(ValueError, match="Invalid coefficient type.*nonexistent"):
        O.expand_coefficients(4, "nonexistent")
    assert O.expand_coefficients(10, "polar_express")[-2:] == [O.COEFFICIENT_SETS["polar_express"][-1]] * 2


# ---------------------------------------------------------------- bf16 rounding
def test_round_to_bf16_against_definition():
    # brute force: nearest representable (8 significant bits), ties to the even mantissa
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(2000).astype(np.float32),
        np.float32([1.0, 1.00390625, 1.01171875, 257.0, 255.0, 0.0, -0.0, 3.0e38, 1e-40]),
        np.float32([1 + 2**-8, 1 + 3 * 2**-8]),  # exact ties: go to even (1.0 and 1 + 2^-6)
    ])
    got = O.round_to_bf16(vals)
    for v, g in zip(vals.astype(np.float64), got.astype(np.float64)):
        if v == 0 or not np.isfinite(v):
            continue
        e = math.floor(math.log2(abs(v)))
        ulp = 2.0 ** (e - 7)
        lo = math.floor(v / ulp) * ulp
        hi = lo + ulp
        if abs(v - lo) < abs(hi - v):
            want = lo
        elif abs(v - lo) > abs(hi - v):
            want = hi
        else:
            want = lo if (round(lo / ulp) % 2 == 0) else hi
        if abs(want) < 2.0**-126 or abs(want) > 3.38e38:
            continue  # subnormal / overflow corner: not exercised by this path
        assert g == want, (v, g, want)
    assert O.round_to_bf16(np.float32([1 + 2**-8]))[0] == 1.0
    assert O.round_to_bf16(np.float32([1 + 3 * 2**-8]))[0] == np.float32(1 + 2**-6)
    assert np.isnan(O.round_to_bf16(np.float32([np.nan]))[0])


# ---------------------------------------------------------------- SYRK / GEMM by brute force
def _loops_syrk(a, c, alpha, beta):
    n, k = a.shape
    out = [[0.0] * n for _ in range(n)]
    for i in range(n):
        for j in range(n):
            s = 0.0
            for p in range(k):
                s += float(a[i, p]) * float(a[j, p])
            out[i][j] = alpha * s + (beta * float(c[i, j]) if c is not None else 0.0)
    return np.array(out)


@pytest.mark.parametrize("n,k", [(5, 7), (8, 3)])
def test_syrk_brute_force_integers(n, k):
    rng = np.random.default_rng(n * 100 + k)
    a = rng.integers(-3, 3, (n, k)).astype(np.float32)
    np.testing.assert_array_equal(O.syrk(a), _loops_syrk(a, None, 1.0, 0.0))
    s = rng.integers(-3, 3, (n, n)).astype(np.float32)
    s = s + s.T
    want = _loops_syrk(s, s, 0.25, 0.5)  # all values are multiples of 1/4 below 2^8: exact in bf16
    np.testing.assert_array_equal(O.syrk(s, s, alpha=0.25, beta=0.5), O.round_to_bf16(want.astype(np.float32)))
    assert np.array_equal(O.syrk(a), O.syrk(a).T)


def test_gemm_axpy_brute_force_integers():
    rng = np.random.default_rng(7)
    bm = rng.integers(-2, 3, (6, 6)).astype(np.float32)
    x = rng.integers(-2, 3, (6, 9)).astype(np.float32)
    want = np.zeros((6, 9))
    for i in range(6):
        for j in range(9):
            want[i, j] = 0.5 * x[i, j] + 0.25 * sum(float(bm[i, p]) * float(x[p, j]) for p in range(6))
    np.testing.assert_array_equal(O.gemm_axpy(bm, x, 0.25, 0.5, round_bf16=False), want)


# ---------------------------------------------------------------- Newton-Schulz against the SVD closed form
@pytest.mark.parametrize("shape", [(48, 48), (64, 32), (32, 64), (3, 24, 40)])
@pytest.mark.parametrize("kind,steps", [("quintic", 5), ("simple", 5), ("polar_express", 9), ("cans", 9), ("deepseekv4", 10), ("cubic5", 5), ("aol", 6)])
def test_newton_schulz_matches_svd_closed_form(shape, kind, steps):
    rng = np.random.default_rng(hash((shape, kind)) % 2**32)
    x = rng.standard_normal(shape).astype(np.float32)
    coeffs = O.expand_coefficients(steps, kind)
    got64 = O.newton_schulz(x, steps, kind, compute_dtype=np.float64)
    if x.ndim == 2:
        want = O.svd_polynomial(x, coeffs)
    else:
        want = np.stack([O.svd_polynomial(x[i], coeffs) for i in range(x.shape[0])])
    # float64 loop vs float64 closed form: agreement far below any tolerance used downstream
    np.testing.assert_allclose(got64, want, atol=2e-6, rtol=0)
    got32 = O.newton_schulz(x, steps, kind)
    np.testing.assert_allclose(got32, want, atol=5e-5, rtol=0)


def test_known_answers_scalar_recurrence():
    for case, x, want in known_answer_cases():
        got = O.newton_schulz(x, case["steps"], case["coefficient_type"])
        np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)
        assert np.array_equal(got == 0, want == 0)


def test_custom_coefficients_and_step_formula():
    rng = np.random.default_rng(3)
    x = (2.0 ** rng.integers(-10, -5, (33, 65))).astype(np.float32)
    sets = [(3.0, 5.0, 7.0), (11.0, 13.0, 17.0)]
    got = O.newton_schulz(x, 2, "custom", custom_coefficient_sets=sets, compute_dtype=np.float64)
    np.testing.assert_allclose(got, O.svd_polynomial(x, sets), rtol=1e-4, atol=1e-7)
    # cubic single step: a x + b (x x^T) x, written independently
    xs = (x / np.linalg.norm(x)).astype(np.float64)
    cub = O.newton_schulz_step(xs, 2.0, -1.5, 0.0)
    np.testing.assert_allclose(cub, 2.0 * xs - 1.5 * (xs @ xs.T) @ xs, atol=1e-14)


def test_transpose_equivariance_and_steps_zero():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((40, 24)).astype(np.float32)
    np.testing.assert_allclose(O.newton_schulz(x.T.copy(), 5), O.newton_schulz(x, 5).T, atol=1e-6)
    np.testing.assert_allclose(O.newton_schulz(x, 0, "quintic"), x / np.linalg.norm(x), rtol=1e-6)


def test_normalisation_underflow_semantics():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((64, 64)) * 1e-30).astype(np.float32)
    assert np.sum(x * x, dtype=np.float32) == 0  # float32 squares underflow
    norm64 = np.sqrt(np.sum(x.astype(np.float64) ** 2))
    assert norm64 != 0
    np.testing.assert_allclose(O.newton_schulz(x, 0, normalize_in_double=True), x / norm64, rtol=1e-6)
    # float32 path: norm 0 -> clamped to eps
    np.testing.assert_allclose(O.frobenius_normalize(x, eps=1e-15), x / np.float32(1e-15), rtol=1e-6)


def test_invariants_quality():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((96, 160)).astype(np.float32)
    out = O.newton_schulz(x, 16, "polar_express").astype(np.float64)
    np.testing.assert_allclose(out @ out.T, np.eye(96), atol=1e-5)
    s = np.linalg.svd(O.newton_schulz(x, 5, "simple"), compute_uv=False)
    assert 0.6 < s.min() and s.max() < 1.2
    u, _, vt = np.linalg.svd(x.astype(np.float64), full_matrices=False)
    np.testing.assert_allclose(O.newton_schulz(x, 5, "quintic"), u @ vt, atol=0.35)  # loose: quintic only lands near 1


def test_bf16_schedule_is_close_to_fp32_and_exact_on_integers():
    rng = np.random.default_rng(13)
    x = rng.standard_normal((64, 128)).astype(np.float32)
    hi = O.newton_schulz(x, 5, "simple")
    med = O.newton_schulz(x, 5, "simple", precision="medium")
    assert np.linalg.norm(med - hi) / np.linalg.norm(hi) < 2e-2
    # integer input, power-of-two coefficients: every pre-rounding value is exact in float32, so the
    # bf16 step must equal a float64 restatement that rounds the three products explicitly.
    xi = rng.integers(-2, 3, (32, 64)).astype(np.float32)
    a, b, c = 2**-1, 2**-2, 2**-3
    r = lambda v: O.round_to_bf16(v.astype(np.float32)).astype(np.float64)
    x64 = xi.astype(np.float64)
    gram = r(x64 @ x64.T)
    poly = r(c * (gram @ gram) + b * gram)
    want = r(a * x64 + poly @ x64)
    np.testing.assert_array_equal(O.newton_schulz_step(xi, a, b, c, bf16=True), want)


def test_shifted_schedule_model_is_the_same_iteration():
    """The diagonal-shift schedule is an exact rewriting: in float64 without rounding it must reproduce the
    plain iteration, and with bf16 rounding it must sit closer to float32 than the reference's schedule."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((96, 160)).astype(np.float32)
    for kind in ("simple", "quintic", "cubic5"):
        hi = O.newton_schulz(x, 5, kind, compute_dtype=np.float64)
        shifted = O.newton_schulz_shifted_bf16(x, 5, kind)
        plain = O.newton_schulz(x, 5, kind, precision="medium")
        e_shift = np.linalg.norm(shifted - hi) / np.linalg.norm(hi)
        e_plain = np.linalg.norm(plain - hi) / np.linalg.norm(hi)
        assert e_shift < 8e-3 and e_shift < e_plain + 5e-4, (kind, e_shift, e_plain)
    # algebra check without any rounding: substitute identity for round_to_bf16
    saved = O.round_to_bf16
    try:
        O.round_to_bf16 = lambda v: np.asarray(v, dtype=np.float32)
        exact = O.newton_schulz_shifted_bf16(x, 5, "simple")
    finally:
        O.round_to_bf16 = saved
    np.testing.assert_allclose(exact, O.newton_schulz(x, 5, "simple"), atol=3e-6)
    # the same for steps taken two at a time on one Gram matrix (pairs of commuting polynomials)
    assert O.pair_schedule([(1, 1, 1)] * 5, True) == [2, 1, 2] and O.pair_schedule([(1, 1, 1)] * 8, True) == [2, 1, 2, 1, 2]
    assert O.pair_schedule([(1, 1, 1)] * 4, True) == [2, 1, 1] and O.pair_schedule([(1, 1, 0)] * 3, True) == [1, 1, 1]
    assert O.pair_schedule([(1, 1, 1)] * 5, False) == [1] * 5
    simple, pe = [(3.4445, -4.7750, 2.0315)], O.expand_coefficients(8, "polar_express")
    assert O.group_schedule(simple * 5, 2) == [3, 2] and O.group_schedule(simple * 8, 2) == [3, 2, 1, 2]
    assert O.group_schedule(simple * 4, 2) == [2, 1, 1] and O.group_schedule(simple * 6, 2) == [3, 2, 1]
    assert O.group_schedule(pe[:5], 2) == [2, 1, 2]  # (a_1 a_2)^2 = 1113: no three steps at once
    assert O.group_schedule(O.expand_coefficients(5, "quintic"), 2) == [3, 2]
    wide = rng.standard_normal((64, 256)).astype(np.float32)
    for kind, steps in (("simple", 5), ("quintic", 5), ("polar_express", 8), ("cubic5", 5)):
        try:
            O.round_to_bf16 = lambda v: np.asarray(v, dtype=np.float32)
            exact = O.newton_schulz_shifted_bf16(wide, steps, kind, pairs=True)
            exact3 = O.newton_schulz_shifted_bf16(wide, steps, kind, pairs=2)
        finally:
            O.round_to_bf16 = saved
        np.testing.assert_allclose(exact, O.newton_schulz(wide, steps, kind), atol=2e-5)
        np.testing.assert_allclose(exact3, O.newton_schulz(wide, steps, kind), atol=3e-5)
        hi = O.newton_schulz(wide, steps, kind, compute_dtype=np.float64)
        e_pair = np.linalg.norm(O.newton_schulz_shifted_bf16(wide, steps, kind, pairs=True) - hi) / np.linalg.norm(hi)
        e_single = np.linalg.norm(O.newton_schulz_shifted_bf16(wide, steps, kind, pairs=False) - hi) / np.linalg.norm(hi)
        assert e_pair < 8e-3 and e_pair < e_single + 1e-3, (kind, e_pair, e_single)
    # scalar known answers: no worse than the reference's bf16 schedule (tiny matrices with singular values
    # spread over 2^-6 .. 1 are hard for any bf16 schedule, hence the comparison instead of a fixed bound)
    fro = lambda g, w: np.linalg.norm(g - w) / np.linalg.norm(w)
    for case, xk, want in known_answer_cases():
        got = O.newton_schulz_shifted_bf16(xk, case["steps"], case["coefficient_type"])
        plain = O.newton_schulz(xk, case["steps"], case["coefficient_type"], precision="medium")
        assert np.array_equal(got == 0, want == 0)
        assert fro(got, want) <= 1.3 * fro(plain, want) + 2e-3


# ---------------------------------------------------------------- Muon pieces
@pytest.mark.parametrize("sizes", [(512, 512), (512, 256), (256, 512), (97, 37), (37, 97)])
def test_scale_factor(sizes):
    o, i = sizes
    assert O.muon_scale_factor(o, i, "shape_scaling") == math.sqrt(max(1, o / i))
    assert O.muon_scale_factor(o, i, "spectral") == math.sqrt(max(o, i))
    assert O.muon_scale_factor(o, i, "unit_rms_norm") == math.sqrt(o / i)
    with pytest.raises(ValueError, match="Invalid mode.*bad"):
        O.muon_scale_factor(o, i, "bad")


def test_optimizer_step_equals_textbook_sgd():
    rng = np.random.default_rng(17)
    p = rng.integers(-5, 5, (7, 9)).astype(np.float32)
    g = rng.integers(-5, 5, (7, 9)).astype(np.float32)
    buf = np.zeros_like(p)
    # momentum 0, decoupled wd: p <- p - lr*wd*p - lr*g   (torch.optim.SGD with weight_decay, on integer data)
    new_p, _ = O.optimizer_step(p, g, buf, lr=2.0, momentum=0.0, weight_decay=0.5)
    np.testing.assert_array_equal(new_p, p - 2.0 * (g + 0.5 * p))
    # EMA momentum (lr 2, beta .5) == classic momentum (lr 1, mu .5) over several steps
    p1, b1 = p.copy(), np.zeros_like(p)
    p2, v2 = p.copy(), np.zeros_like(p)
    for _ in range(5):
        g = rng.integers(-5, 5, (7, 9)).astype(np.float32)
        p1, b1 = O.optimizer_step(p1, g, b1, lr=2.0, momentum=0.5, weight_decay=0.0, weight_decay_method="l2")
        v2 = 0.5 * v2 + g
        p2 = p2 - 1.0 * v2
    np.testing.assert_array_equal(p1, p2)
    ind, _ = O.optimizer_step(p, g, buf, lr=0.0, momentum=0.0, weight_decay=0.25, weight_decay_method="independent")
    np.testing.assert_array_equal(ind, 0.75 * p)


def test_tri_decode_bijection():
    T = 37
    seen = {O.tri_decode(pid) for pid in range(T * (T + 1) // 2)}
    assert seen == {(i, j) for i in range(T) for j in range(i + 1)}
    assert O.tri_decode(0) == (0, 0) and O.tri_decode(2) == (1, 1) and O.tri_decode(3) == (2, 0)
    for pid in (10**6, 2**31 - 1):
        i, j = O.tri_decode(pid)
        assert 0 <= j <= i and i * (i + 1) // 2 + j == pid


def test_torch_cpu_restatement_matches_oracle():
    import torch

    from oracle import ns_torch_cpu

    torch.set_float32_matmul_precision("highest")
    for shape in [(96, 160), (160, 96)]:
        x = torch.randn(*shape)
        coeffs = O.expand_coefficients(5, "simple")
        got = ns_torch_cpu.newton_schulz_cpu(x, coeffs).numpy()
        np.testing.assert_allclose(got, O.newton_schulz(x.numpy(), 5, "simple"), atol=2e-6)
    cub = ns_torch_cpu.newton_schulz_cpu(x, O.expand_coefficients(5, "cubic5")).numpy()
    np.testing.assert_allclose(cub, O.newton_schulz(x.numpy(), 5, "cubic5"), atol=2e-6)


def test_tri_block_decode_bijection():
    for T in [1, 2, 5, 6, 7, 11, 12, 13, 16, 22, 23, 40]:
        seen = {O.tri_block_decode(s, T) for s in range(T * (T + 1) // 2)}
        assert seen == {(i, j) for i in range(T) for j in range(i + 1)}, T
