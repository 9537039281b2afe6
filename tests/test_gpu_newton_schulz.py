"""GPU parity tests of the Newton-Schulz path: step functions, the fused driver and Muon.step().

Tolerance for the bf16 path against float32 Newton-Schulz: relative Frobenius error <= 1e-2
(stated target of this build); tighter bounds apply against the oracle's bf16 schedule.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn

from emerging_optimizers import hip_kernels, utils
from emerging_optimizers.orthogonalized_optimizers import muon, muon_utils
from oracle import ns_oracle as O

from _helpers import known_answer_cases, llama_grad, ns_fp32_torch, rel_fro

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
TOL_FP32 = 1e-2
SIMPLE5 = [(3.4445, -4.7750, 2.0315)] * 5


def _np(t):
    return t.float().cpu().numpy()


# ---------------------------------------------------------------- step functions
def _torch_step(x, a, b, c):
    """The operator sequence of the reference's GEMM steps (muon_utils.py:370-377, 403-410 there) with its rounding
    points on bf16 operands -- every product accumulated in float32 and rounded to bf16 once -- spelled out on torch's
    float32 matmuls: `X @ X.mT`, `addmm(A, A, A, alpha=c, beta=b)`, `addmm(X, B, X, alpha=1, beta=a)` each become a
    float32 product of the bf16 values followed by `.to(bfloat16)`.  (torch's own bf16 matmuls are not used as the
    reference here: the float32 ones with "highest" precision give the same rounding points and an exact sum on the
    integer cases.)  float32 input: plain float32 arithmetic."""
    prev = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("highest")
    try:
        rnd = (lambda t: t.to(BF).float()) if x.dtype == BF else (lambda t: t)
        X = x.float()
        A = rnd(X @ X.mT)
        if c == 0.0:
            return rnd(a * X + b * (A @ X)).to(x.dtype)
        B = rnd(b * A + c * (A @ A))
        return rnd(a * X + B @ X).to(x.dtype)
    finally:
        torch.set_float32_matmul_precision(prev)


@pytest.fixture
def kernel_calls(monkeypatch):
    """Counts the products that reach the HIP kernels through the step functions."""
    calls = {"syrk": 0, "gemm": 0}
    real_gemm = hip_kernels.gemm_axpy
    real = {"tsyrk_ex": muon_utils.triton_kernels.tsyrk_ex, "batched_tsyrk_ex": muon_utils.triton_kernels.batched_tsyrk_ex}

    def counted(kind, fn):
        def run(*args, **kw):
            calls[kind] += 1
            return fn(*args, **kw)

        return run

    monkeypatch.setattr(hip_kernels, "gemm_axpy", counted("gemm", real_gemm))
    for name, fn in real.items():
        monkeypatch.setattr(muon_utils.triton_kernels, name, counted("syrk", fn))
    return calls


# the integer cases of the reference's own step tests (tests/test_muon_utils.py:503-524 there)
@pytest.mark.parametrize("shape", [(32, 32), (32, 64), (2, 32, 32), (4, 32, 64), (8, 16, 128)])
def test_gemm_and_tsyrk_steps_bit_equal_to_torch_and_oracle(gpu, kernel_calls, shape):
    x = torch.randint(-2, 3, shape, device=gpu).to(BF)
    a, b, c = 2**-1, 2**-2, 2**-3
    batched = len(shape) == 3
    tsyrk = muon_utils.batched_newton_schulz_step_tsyrk if batched else muon_utils.newton_schulz_step_tsyrk
    gemm = muon_utils.batched_newton_schulz_step if batched else muon_utils.newton_schulz_step
    got = tsyrk(x, a, b, c)
    assert kernel_calls == {"syrk": 2, "gemm": 1}
    via_gemm_step = gemm(x, a, b, c)
    assert kernel_calls == {"syrk": 4, "gemm": 2}  # the GEMM step runs on the HIP kernels as well
    assert got.dtype == BF and torch.equal(got, via_gemm_step)
    assert torch.equal(got, _torch_step(x, a, b, c))  # float32 torch matmuls with the same rounding points: exact sums
    assert np.array_equal(_np(got), O.newton_schulz_step(_np(x), a, b, c, bf16=True))
    if batched:
        per = torch.stack([muon_utils.newton_schulz_step(x[i], a, b, c) for i in range(shape[0])])
        assert torch.equal(via_gemm_step, per)
    for step in (tsyrk, gemm):  # cubic form: one lower-triangle product, one GEMM
        cubic = step(x, 2.0, -0.5, 0.0)
        assert np.array_equal(_np(cubic), O.newton_schulz_step(_np(x), 2.0, -0.5, 0.0, bf16=True))
        assert torch.equal(cubic, _torch_step(x, 2.0, -0.5, 0.0))
    # an operand stored transposed (what a tall parameter is after the `.mT` view of the driver)
    xt = x.mT.contiguous().mT
    assert not xt.is_contiguous() and torch.equal(gemm(xt, a, b, c), got)


@pytest.mark.parametrize("shape", [(1024, 2048), (2, 1024, 1280), (256, 768), (4, 128, 1024), (2048, 1024)])
def test_gemm_step_on_the_kernels_matches_torch_operators(gpu, kernel_calls, shape):
    """Sizes that reach the direct-to-LDS kernels: random operands, so the float32 sums differ in order from a
    library's and a bf16 rounding flips here and there -- agreement to bf16 resolution with the same rounding points
    computed on float32 matmuls, as the reference asks of its own SYRK against cuBLAS (rtol 0.05 in
    tests/test_triton_kernels.py:138-204 there), and much tighter in norm."""
    x = torch.randn(*shape, device=gpu)
    x = (x / x.norm(dim=(-2, -1), keepdim=True)).to(BF)
    if shape[-2] > shape[-1]:
        x = x.mT  # the driver iterates on the wide orientation: the operand of the step is a transposed view
    step = muon_utils.batched_newton_schulz_step if x.ndim == 3 else muon_utils.newton_schulz_step
    a, b, c = 3.4445, -4.7750, 2.0315
    got = step(x, a, b, c)
    assert kernel_calls == {"syrk": 2, "gemm": 1}
    ref = _torch_step(x.contiguous(), a, b, c)  # the rounding points of the reference's bf16 step
    assert got.shape == ref.shape and got.dtype == BF
    assert rel_fro(got.float().cpu(), ref.float().cpu()) <= 3e-3
    exact = _torch_step(x.float(), a, b, c)  # float32 arithmetic on the same bf16 operand, no rounding in between
    assert rel_fro(got.float().cpu(), exact.cpu()) <= 1.2 * rel_fro(ref.float().cpu(), exact.cpu()) + 1e-4


def test_gemm_step_keeps_torch_for_what_the_kernels_do_not_take(gpu, kernel_calls):
    """float32 operands, dims that are not multiples of 8, rows that are neither contiguous nor transposed-contiguous and
    CPU tensors stay on torch's matmuls (the reference's path); nothing reaches the kernels."""
    for x in (torch.randn(64, 128, device=gpu), torch.randn(12, 40, device=gpu).to(BF), torch.randn(2, 12, 40, device=gpu).to(BF),
              torch.randn(16, 32).to(BF), torch.randn(64, 128, device=gpu).to(BF)[::2]):
        step = muon_utils.batched_newton_schulz_step if x.ndim == 3 else muon_utils.newton_schulz_step
        got = step(x, 0.5, 0.25, 0.125)
        assert got.dtype == x.dtype and got.shape == x.shape
        # (torch's own matmuls against the same rounding points on float32 matmuls: equal up to the order of the sums)
        assert rel_fro(got.float().cpu(), _torch_step(x, 0.5, 0.25, 0.125).float().cpu()) <= 1e-2
    assert kernel_calls == {"syrk": 0, "gemm": 0}


@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (3, 128, 384), (1024, 2560), (4, 128, 1024)])
def test_default_flags_take_the_single_call_driver(gpu, monkeypatch, shape):
    """`newton_schulz(..., use_syrk=False)` -- the reference's default -- on GPU float32 input under "medium": the same
    single library call as with use_syrk=True, bit for bit; and the per-step loop (forced here by replacing a step
    function) reaches the kernels through the GEMM step functions."""
    x = torch.randn(*shape, device=gpu)
    calls = []
    real = hip_kernels.fused_newton_schulz
    monkeypatch.setattr(hip_kernels, "fused_newton_schulz", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    with utils.fp32_matmul_precision("medium"):
        default = muon_utils.newton_schulz(x, steps=5)
        syrk = muon_utils.newton_schulz(x, steps=5, use_syrk=True)
    assert len(calls) == 2 and torch.equal(default, syrk)
    assert rel_fro(default.cpu(), O.newton_schulz(x.cpu().numpy(), 5, "quintic")) <= TOL_FP32
    # "highest": float32 arithmetic on torch, as in the reference
    with utils.fp32_matmul_precision("highest"):
        hi = muon_utils.newton_schulz(x, steps=5)
    assert len(calls) == 2
    assert rel_fro(hi.cpu(), O.newton_schulz(x.cpu().numpy(), 5, "quintic")) <= 1e-4


def test_stepwise_loop_with_default_flags_runs_on_the_kernels(gpu, monkeypatch, kernel_calls):
    x = torch.randn(256, 512, device=gpu)
    original = muon_utils.newton_schulz_step
    seen = []
    monkeypatch.setattr(muon_utils, "newton_schulz_step", lambda X, a, b, c, tp_group=None: (seen.append(X.dtype), original(X, a, b, c, tp_group))[1])
    with utils.fp32_matmul_precision("medium"):
        out = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple")
    assert seen == [BF] * 5 and kernel_calls == {"syrk": 10, "gemm": 5}
    want = O.newton_schulz(x.cpu().numpy(), 5, "simple", precision="medium")  # the reference's bf16 rounding schedule
    assert rel_fro(out.cpu(), want) < 6e-3


# ---------------------------------------------------------------- fused driver, small shapes vs the numpy oracle
# (4, 128, 1024), (2, 256, 1536) and (1536, 256) take the split-K Gram path of short, wide matrices
@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (64, 64), (8, 16), (3, 128, 384), (2, 384, 128), (1024, 1280),
                                   (4, 128, 1024), (2, 256, 1536), (1536, 256)])
@pytest.mark.parametrize("kind,steps", [("simple", 5), ("quintic", 5), ("cubic5", 5), ("polar_express", 8)])
def test_fused_matches_oracle(gpu, shape, kind, steps):
    x = torch.randn(*shape)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x.to(gpu), steps=steps, coefficient_type=kind, use_syrk=True)
    assert got.dtype == torch.float32 and got.shape == x.shape and got.is_contiguous()
    want32 = O.newton_schulz(x.numpy(), steps, kind)
    # 1e-2 is the target for real parameter shapes; a matrix with a handful of rows has no averaging over
    # the rounding errors of its few singular directions (the reference's bf16 path shows the same there).
    tol = TOL_FP32 if min(shape[-2:]) >= 64 else 3e-2
    assert rel_fro(got.cpu(), want32) <= tol
    # Against the CPU model of the driver's own rounding schedule the agreement is much tighter: only the
    # summation order inside the products differs (a rounding flips on a small fraction of entries).
    model = O.newton_schulz_shifted_bf16(x.numpy(), steps, kind)
    assert rel_fro(got.cpu(), model) <= 1e-3 * steps + 1e-3  # flipped roundings accumulate with the step count
    # ... and that schedule beats the reference's bf16 schedule against float32
    ref_sched = O.newton_schulz(x.numpy(), steps, kind, precision="medium")
    assert rel_fro(got.cpu(), want32) <= rel_fro(ref_sched, want32) + 1e-3


@pytest.fixture
def forced_pairs(mi_option):
    """Makes the driver take steps two at a time on one Gram matrix wherever its kernels allow it (by itself it
    does so only for matrices with at least 1024 rows and twice as many columns)."""
    mi_option("ns_pairs", 2)


# (1024, 2048) and (2, 1024, 2304) pair up by the driver's own rule (no override needed)
@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (64, 64), (8, 16), (3, 128, 384), (200, 456), (1024, 1280),
                                   (1024, 2048), (2, 1024, 2304)])
@pytest.mark.parametrize("kind,steps", [("simple", 5), ("quintic", 5), ("quintic", 4), ("cubic5", 5), ("polar_express", 8)])
def test_paired_steps_match_oracle(gpu, forced_pairs, shape, kind, steps):
    x = torch.randn(*shape)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x.to(gpu), steps=steps, coefficient_type=kind, use_syrk=True)
    want32 = O.newton_schulz(x.numpy(), steps, kind)
    tol = TOL_FP32 if min(shape[-2:]) >= 64 else 3e-2
    near_square = max(shape[-2:]) < 2 * min(shape[-2:])
    if near_square:
        tol = max(tol, 1.3e-2)  # outside the driver's own rule: pairs cost accuracy there
    assert rel_fro(got.cpu(), want32) <= tol
    model = O.newton_schulz_shifted_bf16(x.numpy(), steps, kind, pairs=True)
    # (a nearly square random matrix has singular values close to zero, which amplify every flipped rounding)
    assert rel_fro(got.cpu(), model) <= (2.5e-3 if near_square else 1e-3) * steps + 1e-3
    if kind != "cubic5":  # cubic steps never pair: the override must then change nothing, else it must
        single = O.newton_schulz_shifted_bf16(x.numpy(), steps, kind, pairs=False)
        assert rel_fro(model, single) > 1e-5


PAIRS_OPTION = {None: -1, "auto": -1, "0": 0, "pairs": 1, "force": 2}  # values of the library option "ns_pairs"


def test_group_rule_by_shape(gpu, mi_option):
    """Wide matrices take 5 quintic steps as 3 + 2 by default, as 2 + 1 + 2 with the option ns_pairs = 1, one at a time
    with ns_pairs = 0; every variant stays within tolerance and follows its rounding model."""
    x = torch.randn(1024, 2560)
    want32 = O.newton_schulz(x.numpy(), 5, "quintic")
    outs = {}
    for env, mode in ((None, 2), ("pairs", 1), ("0", 0)):
        mi_option("ns_pairs", PAIRS_OPTION[env])
        with utils.fp32_matmul_precision("medium"):
            outs[env] = muon_utils.newton_schulz(x.to(gpu), steps=5, coefficient_type="quintic", use_syrk=True).cpu()
        assert rel_fro(outs[env], want32) <= TOL_FP32
        assert rel_fro(outs[env], O.newton_schulz_shifted_bf16(x.numpy(), 5, "quintic", pairs=mode)) <= 6e-3
    assert rel_fro(outs[None], O.newton_schulz_shifted_bf16(x.numpy(), 5, "quintic")) <= 6e-3  # the model's own rule
    assert not torch.equal(outs[None], outs["pairs"]) and not torch.equal(outs["pairs"], outs["0"])
    # polar_express opens with a large coefficient: no three steps at once there
    mi_option("ns_pairs", -1)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x.to(gpu), steps=5, coefficient_type="polar_express", use_syrk=True).cpu()
    assert rel_fro(got, O.newton_schulz_shifted_bf16(x.numpy(), 5, "polar_express", pairs=1)) <= 6e-3


@pytest.mark.parametrize("shape", [(256, 512), (2, 128, 1024), (1024, 2048), (512, 256), (2, 1000, 504), (2048, 1024)])
def test_deferred_normalisation_is_scale_invariant(gpu, shape):
    """The input is cast to bf16 unnormalised and 1/norm enters the first products; norms outside
    [1e-10, 1e10] take the normalising pass instead.  Powers of two commute with every rounding, so inside
    either regime the result does not depend on the scale at all, and across regimes only by rounding."""
    x = torch.randn(*shape)
    want32 = O.newton_schulz(x.numpy(), 5, "quintic")
    outs = {}
    for k in (0, -20, 20, -45, 50):
        with utils.fp32_matmul_precision("medium"):
            outs[k] = muon_utils.newton_schulz((x * 2.0**k).to(gpu), steps=5, coefficient_type="quintic", use_syrk=True).cpu()
        assert rel_fro(outs[k], want32) <= TOL_FP32, k
    assert torch.equal(outs[0], outs[-20]) and torch.equal(outs[0], outs[20])  # deferred regime
    assert torch.equal(outs[-45], outs[50])                                     # normalising regime
    assert not torch.equal(outs[0], outs[50])


def _spectrum_cases():
    g = torch.Generator().manual_seed(3)
    m, n = 1024, 2560
    u, _ = torch.linalg.qr(torch.randn(m, m, generator=g))
    v, _ = torch.linalg.qr(torch.randn(n, m, generator=g))
    k = torch.arange(1, m + 1, dtype=torch.float32)
    yield "flat power law", (u * k**-0.5) @ v.mT
    yield "steep power law", (u * k**-1.0) @ v.mT
    yield "rank 64 + 10% noise", torch.randn(m, 64, generator=g) @ torch.randn(64, n, generator=g) / 8 + 0.1 * torch.randn(m, n, generator=g)
    yield "gaussian", torch.randn(m, n, generator=g)


@pytest.mark.parametrize("kind", ["simple", "quintic", "aol", "polar_express"])
def test_grouped_steps_are_as_accurate_as_single_steps(gpu, mi_option, kind):
    """Ill-conditioned inputs are far from float32 under any bf16 schedule (the reference's included); what must
    hold is that taking steps in groups (the driver's own rule: 3 + 2 or 2 + 1 + 2; pairs only) does not add to
    that."""
    for name, x in _spectrum_cases():
        want32 = O.newton_schulz(x.numpy(), 5, kind, compute_dtype=np.float64)
        err = {}
        for env in ("auto", "pairs", "0"):
            mi_option("ns_pairs", PAIRS_OPTION[env])
            with utils.fp32_matmul_precision("medium"):
                got = muon_utils.newton_schulz(x.to(gpu), steps=5, coefficient_type=kind, use_syrk=True).cpu()
            err[env] = rel_fro(got, want32)
        assert err["auto"] <= 1.15 * err["0"] + 5e-4, (name, kind, err)
        assert err["pairs"] <= 1.15 * err["0"] + 5e-4, (name, kind, err)


def test_fused_known_answers(gpu):
    for case, x, want in known_answer_cases():
        with utils.fp32_matmul_precision("medium"):
            got = muon_utils.newton_schulz(torch.from_numpy(x).to(gpu), steps=case["steps"],
                                           coefficient_type=case["coefficient_type"], use_syrk=True)
        got = got.cpu().numpy().astype(np.float64)
        assert np.array_equal(got == 0, want == 0)  # permutation structure is preserved exactly
        # Every product has a single non-zero term here, so there is no summation-order freedom: the GPU
        # must reproduce the CPU model of its schedule up to fused-multiply-add differences ...
        model = O.newton_schulz_shifted_bf16(x, case["steps"], case["coefficient_type"])
        assert rel_fro(got, model) <= 5e-3
        # ... and be no further from the exact scalar recurrence than the reference's bf16 schedule.
        plain = O.newton_schulz(x, case["steps"], case["coefficient_type"], precision="medium")
        assert rel_fro(got, want) <= 1.3 * rel_fro(plain, want) + 2e-3


def test_fused_semantics(gpu):
    x = torch.randn(64, 128, device=gpu)
    with utils.fp32_matmul_precision("medium"):
        # steps = 0: normalised input, float32, no bf16 rounding
        out0 = muon_utils.newton_schulz(x, steps=0, use_syrk=True)
        torch.testing.assert_close(out0, x / x.norm(), rtol=1e-6, atol=0)
        # float64 norm for tiny inputs (float32 squares underflow)
        tiny = torch.randn(256, 256, device=gpu) * 1e-30
        assert torch.linalg.vector_norm(tiny) == 0
        out = muon_utils.newton_schulz(tiny, steps=0, use_syrk=True, normalize_in_double=True)
        torch.testing.assert_close(out, (tiny.double() / torch.linalg.vector_norm(tiny, dtype=torch.double)).float(), rtol=1e-6, atol=0)
        # all-zero input: eps clamp, no NaN
        z = muon_utils.newton_schulz(torch.zeros(32, 64, device=gpu), steps=5, use_syrk=True)
        assert torch.equal(z, torch.zeros_like(z))
        # input is not modified; 3-D equals per-slice
        keep = x.clone()
        muon_utils.newton_schulz(x, steps=5, use_syrk=True)
        assert torch.equal(x, keep)
        xb = torch.randint(-3, 4, (4, 32, 64), device=gpu).float()
        both = muon_utils.newton_schulz(xb, steps=5, coefficient_type="quintic", use_syrk=True)
        per = torch.stack([muon_utils.newton_schulz(xb[i], steps=5, coefficient_type="quintic", use_syrk=True) for i in range(4)])
        assert torch.equal(both, per)
        # use_syrk on/off agree at the reference's tolerance (test_muon_utils.py:526-532 there)
        ref = muon_utils.newton_schulz(xb, steps=5, coefficient_type="quintic", use_syrk=False)
        torch.testing.assert_close(both, ref, atol=1e-2, rtol=1e-2)
        # transposed (non-contiguous) input view
        xt = torch.randn(128, 64, device=gpu).T
        torch.testing.assert_close(muon_utils.newton_schulz(xt, steps=5, use_syrk=True),
                                   muon_utils.newton_schulz(xt.contiguous(), steps=5, use_syrk=True))


def test_fused_and_stepwise_paths_agree(gpu, monkeypatch):
    """Replacing a step function forces the per-step Python loop (HIP kernel per product); it has to land
    within bf16 noise of the single-call driver."""
    x = torch.randn(256, 512, device=gpu)
    with utils.fp32_matmul_precision("medium"):
        fused = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
        calls = {"n": 0}
        original = muon_utils.newton_schulz_step_tsyrk

        def counting(X, a, b, c, tp_group=None):
            calls["n"] += 1
            return original(X, a, b, c, tp_group=tp_group)

        monkeypatch.setattr(muon_utils, "newton_schulz_step_tsyrk", counting)
        stepwise = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
    assert calls["n"] == 5
    # The step functions keep the reference's rounding points (A and B rounded with their full diagonal),
    # the single-call driver does not; each is within ~1e-2 of float32, so they are within ~2e-2 of each other.
    assert rel_fro(stepwise, fused) < 2e-2
    want = O.newton_schulz(x.cpu().numpy(), 5, "simple", precision="medium")
    assert rel_fro(stepwise.cpu(), want) < 6e-3  # same schedule as the oracle, different summation order


@pytest.mark.parametrize("shape", [(4, 4), (4, 8), (8, 4), (2, 4, 8), (12, 40)])
def test_unaligned_shapes_use_library_gemm_step(gpu, shape, monkeypatch):
    calls = {"n": 0}
    name = "newton_schulz_step" if len(shape) == 2 else "batched_newton_schulz_step"
    original = getattr(muon_utils, name)

    def counting(X, a, b, c, tp_group=None):
        calls["n"] += 1
        return original(X, a, b, c, tp_group=tp_group)

    def forbidden(*args, **kw):
        raise AssertionError("SYRK step must not run for a shape that is not a multiple of 8")

    monkeypatch.setattr(muon_utils, name, counting)
    monkeypatch.setattr(muon_utils, "newton_schulz_step_tsyrk", forbidden)
    monkeypatch.setattr(muon_utils, "batched_newton_schulz_step_tsyrk", forbidden)
    with utils.fp32_matmul_precision("medium"):
        muon_utils.newton_schulz(torch.randn(shape, device=gpu), steps=1, coefficient_type="simple", use_syrk=True)
    assert calls["n"] == 1


def test_gpu_torch_reference_is_trustworthy(gpu):
    """The float32 torch loop used as reference at full size agrees with the numpy oracle at a size both can do."""
    x = torch.randn(384, 640)
    want = O.newton_schulz(x.numpy(), 5, "simple")
    got = ns_fp32_torch(x.to(gpu), SIMPLE5)
    assert rel_fro(got.cpu(), want) < 1e-5


# ---------------------------------------------------------------- benchmark configurations at full size
def _sv_band(out, lo=0.55, hi=1.25):
    """Singular values of the result via the eigenvalues of the small Gram matrix in float64."""
    y = out.double()
    gram = y @ y.mT if y.shape[-2] <= y.shape[-1] else y.mT @ y
    ev = torch.linalg.eigvalsh(gram).clamp_min(0).sqrt()
    return float(ev.min()), float(ev.max())


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 14336), (14336, 4096)])
def test_llama_shapes_within_tolerance(gpu, shape):
    """Llama-3-8B-shaped gradients (N(0, 1e-3^2) with 1 % outliers at 50 sigma), 5 steps."""
    x = llama_grad(shape, seed=shape[1]).to(gpu)
    ref = ns_fp32_torch(x, SIMPLE5)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
    err = rel_fro(got, ref)
    print(f"\n  {shape}: rel_fro vs fp32 = {err:.3e}")
    assert err <= TOL_FP32
    smin, smax = _sv_band(got)
    rmin, rmax = _sv_band(ref)
    print(f"  singular values: got [{smin:.3f}, {smax:.3f}]  fp32 [{rmin:.3f}, {rmax:.3f}]")
    assert abs(smin - rmin) < 0.03 and abs(smax - rmax) < 0.03
    # transpose equivariance: NS(x^T) == NS(x)^T, different kernels (K-strided loaders) underneath
    with utils.fp32_matmul_precision("medium"):
        got_t = muon_utils.newton_schulz(x.T.contiguous(), steps=5, coefficient_type="simple", use_syrk=True)
    assert rel_fro(got_t.T, got) < 5e-3


@pytest.mark.parametrize("shape", [(1024, 2048), (1024, 8192), (2048, 8192), (1536, 4096), (3072, 8192), (2, 2048, 4096),
                                   (8192, 2048), (1000, 2104)])
@pytest.mark.parametrize("kind,steps", [("simple", 5), ("quintic", 5), ("polar_express", 8), ("deepseekv4", 10)])
def test_wide_shapes_grouped_by_default(gpu, shape, kind, steps):
    """Shapes that take several steps per Gram matrix by the driver's own rule (tile edges, batches, tall inputs,
    long schedules: 3+2, 2+1+2+1+2, 3+2+1+2+1+1), against float32 torch on the GPU."""
    x = (torch.randn(*shape, generator=torch.Generator().manual_seed(sum(shape))) * 1e-2).to(gpu)
    coeffs = O.expand_coefficients(steps, kind)
    ref = ns_fp32_torch(x, coeffs)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=steps, coefficient_type=kind, use_syrk=True)
    errs = [rel_fro(got[i], ref[i]) for i in range(shape[0])] if len(shape) == 3 else [rel_fro(got, ref)]
    assert max(errs) <= TOL_FP32, errs


def test_quintic_default_at_headline_shape(gpu):
    x = llama_grad((4096, 14336), seed=7).to(gpu)
    coeffs = muon_utils._COEFFICIENT_SETS["quintic"]
    ref = ns_fp32_torch(x, coeffs)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="quintic", use_syrk=True)
    assert rel_fro(got, ref) <= TOL_FP32


def test_per_head_grouped_launch(gpu):
    """32 independent 128 x 4096 heads in one 3-D call == 32 separate 2-D calls, and within tolerance."""
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(32, 128, 4096, generator=g) * 1e-3).to(gpu)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
        per = torch.stack([muon_utils.newton_schulz(x[i], steps=5, coefficient_type="simple", use_syrk=True) for i in range(32)])
    assert torch.equal(got, per)
    ref = ns_fp32_torch(x, SIMPLE5)
    errs = [rel_fro(got[i], ref[i]) for i in range(32)]
    assert max(errs) <= TOL_FP32


def test_moe_shard_shape_with_per_expert_scales(gpu):
    g = torch.Generator().manual_seed(0)
    scales = torch.exp(torch.empty(8).uniform_(np.log(1e-4), np.log(1e-2), generator=g))
    x = (torch.randn(8, 1792, 4096, generator=g) * scales[:, None, None]).to(gpu)
    ref = ns_fp32_torch(x, SIMPLE5)
    with utils.fp32_matmul_precision("medium"):
        got = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
    assert max(rel_fro(got[i], ref[i]) for i in range(8)) <= TOL_FP32
    # per-matrix normalisation makes the result independent of each expert's scale
    with utils.fp32_matmul_precision("medium"):
        got2 = muon_utils.newton_schulz(x * 4.0, steps=5, coefficient_type="simple", use_syrk=True)
    assert torch.equal(got, got2)


# ---------------------------------------------------------------- Muon on the GPU
def test_muon_use_syrk_matches_library_path(gpu):
    p = nn.Parameter(torch.randint(-5, 5, (32, 32), device=gpu).float())
    q = nn.Parameter(p.detach().clone())
    p.grad = torch.randint_like(p, -5, 5)
    q.grad = p.grad.clone()
    a = muon.Muon([p], num_ns_steps=1, coefficient_type="simple", use_syrk=True)
    b = muon.Muon([q], num_ns_steps=1, coefficient_type="simple", use_syrk=False)
    assert a.use_syrk is True
    a.step()
    b.step()
    torch.testing.assert_close(p.data, q.data)


@pytest.mark.parametrize("shape", [(1024, 1024), (1024, 3584), (3584, 1024)])
def test_muon_step_llama_like(gpu, shape):
    """Momentum 0.95 with Nesterov on a warmed buffer; kernel path vs the same optimizer in float32."""
    lr = 0.02
    w0 = torch.randn(shape, generator=torch.Generator().manual_seed(1)) * 0.02
    p, q = nn.Parameter(w0.clone().to(gpu)), nn.Parameter(w0.clone().to(gpu))
    fast = muon.Muon([p], lr=lr, momentum=0.95, nesterov=True, coefficient_type="simple", use_syrk=True)
    slow = muon.Muon([q], lr=lr, momentum=0.95, nesterov=True, coefficient_type="simple", fp32_matmul_prec="highest")
    for step in range(4):
        g = llama_grad(shape, seed=100 + step).to(gpu)
        p.grad, q.grad = g.clone(), g.clone()
        before = p.detach().clone()
        fast.step()
        slow.step()
        upd_fast = p.detach() - before * (1 - lr * 0.01)
    # the weights drift apart only through the bf16 error of each update: ||dW_fast - dW_slow|| <= 1e-2 ||dW||
    diff = (p.detach() - q.detach()).norm()
    assert float(diff / (4 * upd_fast.norm())) <= TOL_FP32
    # update = -lr sqrt(max(shape)) NS(direction) with ||NS||_F^2 ~ min(shape) (singular values in [0.68, 1.14]):
    # its root mean square is lr times a number close to 1
    rms = float(upd_fast.pow(2).mean().sqrt()) / lr
    assert 0.6 < rms < 1.2


def test_per_head_muon_equivalence(gpu):
    heads, d, n = 8, 128, 1024
    g = torch.randn(heads * d, n, device=gpu)
    fn = muon.Muon([nn.Parameter(torch.zeros(d, n, device=gpu))], use_syrk=True).scaled_orthogonalize_fn
    with utils.fp32_matmul_precision("medium"):
        stacked = fn(g.view(heads, d, n)).reshape(heads * d, n)
        separate = torch.cat([fn(g[i * d:(i + 1) * d]) for i in range(heads)])
    torch.testing.assert_close(stacked, separate, atol=1e-6, rtol=0)


# ---------------------------------------------------------------- one-call Muon update
@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (1024, 1024), (1024, 3584), (3584, 1024)])
@pytest.mark.parametrize("nesterov", [True, False])
def test_fused_muon_update_matches_explicit_statements(gpu, shape, nesterov):
    """mi_muon_update_bf16 against lerp_/lerp + newton_schulz + the two in-place parameter updates."""
    lr, beta, wd = 0.02, 0.95, 0.1
    gen = torch.Generator().manual_seed(7)
    p0 = (torch.randn(shape, generator=gen) * 0.02).to(gpu)
    buf0 = (torch.randn(shape, generator=gen) * 1e-3).to(gpu)
    g = llama_grad(shape, seed=3).to(gpu)
    scale = muon.get_muon_scale_factor(*shape, mode="spectral")
    # statement by statement, as OrthogonalizedOptimizer.step does it
    p_ref, buf_ref = p0.clone(), buf0.clone()
    p_ref.add_(p_ref, alpha=-wd * lr)
    buf_ref.lerp_(g, 1 - beta)
    direction = g.lerp(buf_ref, beta) if nesterov else buf_ref
    with utils.fp32_matmul_precision("medium"):
        update = muon_utils.newton_schulz(direction, steps=5, coefficient_type="simple", use_syrk=True) * scale
    p_ref.add_(update, alpha=-lr)
    # one call
    p, buf = p0.clone(), buf0.clone()
    hip_kernels.fused_muon_update(p, g, buf, SIMPLE5, beta=beta, nesterov=nesterov, param_decay=1 - wd * lr,
                                  update_scale=-lr * scale)
    torch.testing.assert_close(buf, buf_ref, rtol=2e-6, atol=5e-9)  # one ulp of the largest entries (5e-2)
    # the parameter differs only through float32 rounding of the elementwise parts and through bf16 rounding flips
    # of a direction that may differ in the last bit (square matrices amplify those the most): below the 1e-2
    # budget each of the two results has against float32
    assert float((p - p_ref).norm() / (p_ref - p0).norm()) <= 8e-3
    assert float(rel_fro(_np((p - (1 - wd * lr) * p0) / (-lr * scale)), _np(ns_fp32_torch(direction, SIMPLE5)))) <= TOL_FP32


@pytest.mark.parametrize("method,wd", [("decoupled", 0.1), ("independent", 0.01), ("palm", 0.5), ("decoupled", 0.0)])
def test_muon_step_takes_the_fused_update_and_agrees_with_the_statement_path(gpu, monkeypatch, method, wd):
    shape, lr = (512, 1024), 0.02
    w0 = torch.randn(shape, generator=torch.Generator().manual_seed(1)) * 0.02
    p, q = nn.Parameter(w0.clone().to(gpu)), nn.Parameter(w0.clone().to(gpu))
    kw = dict(lr=lr, momentum=0.95, nesterov=True, weight_decay=wd, weight_decay_method=method,
              coefficient_type="simple", use_syrk=True)
    fused, plain = muon.Muon([p], **kw), muon.Muon([q], **kw)
    calls = []
    real = hip_kernels.fused_muon_update
    monkeypatch.setattr(hip_kernels, "fused_muon_update", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    for step in range(3):
        g = llama_grad(shape, seed=200 + step).to(gpu)
        p.grad, q.grad = g.clone(), g.clone()
        fused.step()
        n_calls = len(calls)
        monkeypatch.setattr(muon, "FUSED_MUON_STEP", False)
        plain.step()
        monkeypatch.setattr(muon, "FUSED_MUON_STEP", True)
        assert len(calls) == n_calls == step + 1  # the fused optimizer used the library call, the plain one did not
    torch.testing.assert_close(fused.state[p]["momentum_buffer"], plain.state[q]["momentum_buffer"], rtol=2e-6, atol=5e-9)
    assert float((p.detach() - q.detach()).norm() / (q.detach() - w0.to(gpu)).norm()) <= 8e-3


def test_muon_step_keeps_the_statement_path_when_something_watches_the_update(gpu, monkeypatch):
    calls = []
    real = hip_kernels.fused_muon_update
    monkeypatch.setattr(hip_kernels, "fused_muon_update", lambda *a, **k: (calls.append(1), real(*a, **k))[1])

    class Watching(muon.Muon):
        def pre_weight_update_fn_inplace(self, p, update):
            self.seen = update.shape

    for cls, kw in ((Watching, {}), (muon.Muon, {"weight_decay": 0.1, "weight_decay_method": "l2"}),
                    (muon.Muon, {"fp32_matmul_prec": "highest"})):
        p = nn.Parameter(torch.randn(64, 128, device=gpu))
        p.grad = torch.randn_like(p)
        cls([p], use_syrk=True, **kw).step()
    assert calls == []


@pytest.mark.parametrize("shape", [(32, 128, 4096), (3, 128, 1024), (1, 128, 2048), (5, 4096, 128)])
@pytest.mark.parametrize("coefficient_type", ["simple", "quintic", "polar_express"])
def test_per_head_slab_kernel_against_the_general_kernels(gpu, mi_option, shape, coefficient_type):
    """128-row matrices: the product that ends a group of steps, and the partial Gram matrices of its result, come from
    the slab kernel (inst_head_apply.hip).  The option head_apply = 0 sends the same call through the general GEMM+AXPY kernel
    and a separate Gram kernel.  The two differ in how the sum of squares behind the diagonal shift is split into
    partial sums (one per 512-column slice against one per 256-column tile), i.e. in the last bits of the shift, which
    moves a few bf16 roundings: measured 0 to 6e-5 apart for the "simple" and "quintic" coefficients and up to 2.7e-3
    for "polar_express", whose first step (a = 8.2) amplifies rounding noise most -- inside the distance of either from
    float32, not bit for bit.  A batch entry equals the matrix computed alone, bit for bit."""
    x = torch.randn(*shape, device=gpu, generator=torch.Generator(device=gpu).manual_seed(21)) * 3e-3
    with utils.fp32_matmul_precision("medium"):
        mi_option("head_apply", 1)
        new = muon_utils.newton_schulz(x, steps=5, coefficient_type=coefficient_type, use_syrk=True)
        alone = muon_utils.newton_schulz(x[-1], steps=5, coefficient_type=coefficient_type, use_syrk=True)
        mi_option("head_apply", 0)
        old = muon_utils.newton_schulz(x, steps=5, coefficient_type=coefficient_type, use_syrk=True)
    assert torch.isfinite(new).all()
    diff = rel_fro(new, old)
    print(f"\n  {shape} {coefficient_type}: slab kernel vs general kernels rel_fro = {diff:.2e}")
    assert diff <= (5e-3 if coefficient_type == "polar_express" else 2e-4)
    assert torch.equal(new[-1], alone)


@pytest.mark.parametrize("shape", [(32, 128, 4096), (3, 128, 1024), (1, 128, 2048)])
@pytest.mark.parametrize("magnitude", [3e-3, 1e-17, 1e15])
def test_per_head_input_pass_against_the_general_passes(gpu, mi_option, shape, magnitude):
    """128-row matrices: the pass over the float32 input also leaves the partial Gram matrices of its bf16 copy
    (head_front_kernel in inst_head_apply.hip).  The option head_front = 0 sends the same call through the general sum-of-squares
    pass and a Gram kernel of its own.  The two add the squares in a different order, so the norm may differ in its last
    bit, which moves a few bf16 roundings: the results agree to 2e-4 and either is as far from float32 as the other.
    The magnitudes 1e-17 and 1e15 put the norm outside the range where the divide by it may be left to the consumers:
    the second launch of the input pass then rewrites the copy and its Gram matrices from x / norm.  A batch entry
    equals the matrix computed alone, bit for bit."""
    x = torch.randn(*shape, device=gpu, generator=torch.Generator(device=gpu).manual_seed(33)) * magnitude
    with utils.fp32_matmul_precision("medium"):
        mi_option("head_front", 1)
        new = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
        alone = muon_utils.newton_schulz(x[-1], steps=5, coefficient_type="simple", use_syrk=True)
        mi_option("head_front", 0)
        old = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
    assert torch.isfinite(new).all()
    diff = rel_fro(new, old)
    ref = ns_fp32_torch((x.double() / magnitude).float(), SIMPLE5)  # (the iteration does not depend on the scale of x)
    print(f"\n  {shape} x {magnitude:g}: input pass with Gram partials vs general passes rel_fro = {diff:.2e}; "
          f"vs float32 {rel_fro(_np(new), _np(ref)):.2e} / {rel_fro(_np(old), _np(ref)):.2e}")
    assert diff <= 2e-4
    assert rel_fro(_np(new), _np(ref)) <= TOL_FP32
    assert torch.equal(new[-1], alone)


@pytest.mark.parametrize("nesterov", [True, False])
def test_per_head_input_pass_with_a_momentum_source(gpu, mi_option, nesterov):
    """The fused optimizer update on 128-row matrices: the input pass that leaves the Gram partials also updates the
    momentum buffer and orthogonalises the direction it defines.  Against the same call through the general passes
    (option head_front = 0): the buffer bit for bit (the same elementwise formula), the parameter to rounding noise."""
    shape, lr, beta, wd = (8, 128, 2048), 0.02, 0.95, 0.1
    gen = torch.Generator().manual_seed(11)
    p0 = (torch.randn(shape, generator=gen) * 0.02).to(gpu)
    buf0 = (torch.randn(shape, generator=gen) * 1e-3).to(gpu)
    g = (torch.randn(shape, generator=gen) * 1e-2).to(gpu)
    res = {}
    for front in ("1", "0"):
        mi_option("head_front", int(front))
        p, buf = p0.clone(), buf0.clone()
        hip_kernels.fused_muon_update(p, g, buf, SIMPLE5, beta=beta, nesterov=nesterov, param_decay=1 - wd * lr, update_scale=-lr)
        res[front] = (p, buf)
    buf_ref = buf0.clone().lerp_(g, 1 - beta)
    torch.testing.assert_close(res["1"][1], buf_ref, rtol=2e-6, atol=5e-9)
    assert torch.equal(res["1"][1], res["0"][1])
    assert float((res["1"][0] - res["0"][0]).norm() / (res["0"][0] - p0).norm()) <= 2e-4
    direction = g.lerp(buf_ref, beta) if nesterov else buf_ref
    assert float(rel_fro(_np((res["1"][0] - (1 - wd * lr) * p0) / (-lr)), _np(ns_fp32_torch(direction, SIMPLE5)))) <= TOL_FP32


@pytest.mark.parametrize("shape", [(3584, 1024), (2048, 1024), (512, 256), (2, 2304, 1024), (8, 4096, 1792), (14336, 4096)])
def test_tall_input_result_written_transposed_by_the_last_product(gpu, mi_option, shape):
    """Tall inputs are iterated in the transposed orientation.  Where the last product runs on kernels with the staged
    epilogue, it writes its float32 result transposed, straight into the output; the option tall_direct = 0 restores the
    float32 staging copy and the transposing pass.  Same arithmetic, so the two agree bit for bit -- also for the
    fused optimizer update, where the epilogue reads the parameter it updates in the transposed pattern."""
    gen = torch.Generator(device=gpu).manual_seed(9)
    x = torch.randn(*shape, device=gpu, generator=gen) * 1e-3
    p0 = torch.randn(*shape, device=gpu, generator=gen) * 0.02
    buf0 = torch.randn(*shape, device=gpu, generator=gen) * 1e-3
    res = {}
    for direct in ("1", "0"):
        mi_option("tall_direct", int(direct))
        with utils.fp32_matmul_precision("medium"):
            out = muon_utils.newton_schulz(x, steps=5, coefficient_type="simple", use_syrk=True)
        p, buf = p0.clone(), buf0.clone()
        hip_kernels.fused_muon_update(p, x, buf, SIMPLE5, beta=0.95, nesterov=True, param_decay=0.999, update_scale=-0.02)
        res[direct] = (out, p, buf)
    assert torch.isfinite(res["1"][0]).all()
    for a, b in zip(res["1"], res["0"]):
        assert torch.equal(a, b)
    if shape != (14336, 4096):
        assert rel_fro(_np(res["1"][0]), _np(ns_fp32_torch(x, SIMPLE5))) <= TOL_FP32


@pytest.mark.parametrize("shape", [(32, 128, 4096), (1024, 4096)])
def test_fused_call_replays_from_a_hip_graph(gpu, shape):
    """The single-call driver allocates nothing and records no memset: captured into a HIP graph (its workspace
    allocated beforehand by a warm-up call), every replay -- with eager work of the same library in between -- gives
    the bits of the eager call."""
    x = torch.randn(*shape, device=gpu, generator=torch.Generator(device=gpu).manual_seed(5)) * 1e-3
    other = torch.randn(2048, 2048, device=gpu).to(torch.bfloat16)
    with utils.fp32_matmul_precision("medium"):
        run = lambda: muon_utils.newton_schulz(x, steps=5, coefficient_type="quintic", use_syrk=True)
        eager = run()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = run()
        for _ in range(3):
            out.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
            hip_kernels.tsyrk_ex(other)  # eager work between the replays
            torch.cuda.synchronize()
