"""Which operands of the step functions go to the HIP kernels, and how the three products of a step are wired to
them -- checked on the CPU by standing in for the device test and for the kernels.

The kernels take a bf16 operand on a gfx950 GPU with both dims multiples of 8 that is stored row-major or as its
transpose (reference: the step functions of muon_utils.py:348-476); everything else stays on torch's operators.  The
products of a step on the kernels are `A = syrk(X)`, `B = syrk(A, A, alpha=c, beta=b)`,
`X' = gemm_axpy(B, X, alpha=1, beta=a)` (cubic: `gemm_axpy(A, X, alpha=b, beta=a)`): here the two kernel entry points
are replaced by float32 matmuls with one bf16 rounding per product, and the result must equal the oracle's bf16 step
bit for bit on the integer cases of the reference's own step tests (tests/test_muon_utils.py:503-524 there).
"""
import numpy as np
import pytest
import torch

from emerging_optimizers import hip_kernels
from emerging_optimizers.hip_kernels import newton_schulz as ns_module
from emerging_optimizers.orthogonalized_optimizers import muon_utils
from oracle import ns_oracle as O

BF = torch.bfloat16


@pytest.fixture
def as_if_on_gpu(monkeypatch):
    """CPU tensors pass for tensors on a gfx950 GPU; the library counts as loaded."""
    asked = []
    for where in (hip_kernels, ns_module):  # (the package's name and the one `fused_supported` sees in its own module)
        monkeypatch.setattr(where, "on_kernel_device", lambda t: True)
        monkeypatch.setattr(where, "require_library", lambda: asked.append(1))
    return asked


def test_which_operands_the_kernels_take(as_if_on_gpu):
    take = muon_utils._kernels_take
    x = torch.zeros(16, 32, dtype=BF)
    assert take(x) and take(x.mT) and take(torch.zeros(3, 16, 32, dtype=BF)) and take(torch.zeros(3, 32, 16, dtype=BF).mT)
    assert len(as_if_on_gpu) == 4  # each of them asked for the library
    for other in (torch.zeros(16, 32), torch.zeros(12, 40, dtype=BF), torch.zeros(16, 36, dtype=BF), torch.zeros(32, 32, dtype=BF)[::2],
                  torch.zeros(0, 32, dtype=BF), torch.zeros(16, 32, dtype=torch.float16)):
        assert not take(other)
    assert len(as_if_on_gpu) == 4  # and what stays on torch never does


def test_operands_on_other_devices_stay_on_torch():
    assert not muon_utils._kernels_take(torch.zeros(16, 32, dtype=BF))  # a CPU tensor
    x = torch.randint(-2, 3, (16, 32)).to(BF)
    got = muon_utils.newton_schulz_step(x, 0.5, 0.25, 0.125)
    assert np.array_equal(got.float().numpy(), O.newton_schulz_step(x.float().numpy(), 0.5, 0.25, 0.125, bf16=True))


def test_no_silent_path_when_the_library_is_missing(monkeypatch):
    def missing():
        raise RuntimeError("libmi_ns.so is not built")

    for where in (hip_kernels, ns_module):
        monkeypatch.setattr(where, "on_kernel_device", lambda t: True)
        monkeypatch.setattr(where, "require_library", missing)
    x = torch.zeros(16, 32, dtype=BF)
    for step in (muon_utils.newton_schulz_step, muon_utils.batched_newton_schulz_step):
        with pytest.raises(RuntimeError, match="libmi_ns"):
            step(x if step is muon_utils.newton_schulz_step else x[None], 0.5, 0.25, 0.125)
    # an operand the kernels would not take anyway never asks for the library
    out = muon_utils.newton_schulz_step(torch.zeros(12, 40, dtype=BF), 0.5, 0.25, 0.125)
    assert out.shape == (12, 40)
    with pytest.raises(RuntimeError, match="libmi_ns"):
        hip_kernels.fused_supported(torch.zeros(16, 32))
    assert not hip_kernels.fused_supported(torch.zeros(12, 40)) and not hip_kernels.fused_supported(torch.zeros(16, 32, dtype=BF))


@pytest.fixture
def stand_in_kernels(monkeypatch, as_if_on_gpu):
    """float32 products rounded to bf16 once, behind the signatures of the kernel entry points; records the calls."""
    calls = []

    def syrk(a, c=None, alpha=1.0, beta=0.0, **kw):
        assert a.dtype == BF and not kw
        calls.append(("syrk", tuple(a.shape), c is not None, alpha, beta))
        d = alpha * (a.float() @ a.float().mT)
        if c is not None:
            d = d + beta * c.float()
        return d.to(BF)

    def gemm_axpy(bm, x, alpha=1.0, beta=1.0, **kw):
        assert bm.dtype == BF and x.dtype == BF and not kw
        calls.append(("gemm", tuple(x.shape), alpha, beta))
        return (beta * x.float() + alpha * (bm.float() @ x.float())).to(BF)

    monkeypatch.setattr(muon_utils.triton_kernels, "tsyrk_ex", syrk)
    monkeypatch.setattr(muon_utils.triton_kernels, "batched_tsyrk_ex", syrk)
    monkeypatch.setattr(hip_kernels, "gemm_axpy", gemm_axpy)
    return calls


@pytest.mark.parametrize("shape", [(32, 32), (32, 64), (2, 32, 32), (4, 32, 64), (8, 16, 128)])
def test_products_of_a_step_are_wired_to_the_kernels_as_the_reference_orders_them(stand_in_kernels, shape):
    x = torch.randint(-2, 3, shape, generator=torch.Generator().manual_seed(sum(shape))).to(BF)
    a, b, c = 2**-1, 2**-2, 2**-3
    batched = len(shape) == 3
    steps = ((muon_utils.batched_newton_schulz_step, muon_utils.batched_newton_schulz_step_tsyrk) if batched else
             (muon_utils.newton_schulz_step, muon_utils.newton_schulz_step_tsyrk))
    m = shape[-2]
    gram = shape[:-2] + (m, m)
    for step in steps:
        del stand_in_kernels[:]
        got = step(x, a, b, c)
        assert stand_in_kernels == [("syrk", shape, False, 1.0, 0.0), ("syrk", gram, True, c, b), ("gemm", shape, 1.0, a)]
        assert got.dtype == BF
        assert np.array_equal(got.float().numpy(), O.newton_schulz_step(x.float().numpy(), a, b, c, bf16=True))
        # cubic form: the Gram matrix itself multiplies X
        del stand_in_kernels[:]
        cubic = step(x, 2.0, -0.5, 0.0)
        assert stand_in_kernels == [("syrk", shape, False, 1.0, 0.0), ("gemm", shape, -0.5, 2.0)]
        assert np.array_equal(cubic.float().numpy(), O.newton_schulz_step(x.float().numpy(), 2.0, -0.5, 0.0, bf16=True))


def test_single_call_path_needs_the_default_orientation_untouched_steps_and_no_group(monkeypatch, as_if_on_gpu):
    ok = muon_utils._fused_path_ok
    wide, tall = torch.zeros(16, 32), torch.zeros(32, 16)
    assert ok(wide, False, None) and ok(tall, True, None)
    assert not ok(wide, True, None) and not ok(tall, False, None)  # a forced orientation
    assert not ok(wide, False, object())  # a tensor-parallel group: the Gram matrix is all-reduced between the products
    assert not ok(torch.zeros(12, 40), False, None)
    monkeypatch.setattr(muon_utils, "newton_schulz_step", lambda X, a, b, c, tp_group=None: X)  # a replaced step function
    assert not ok(wide, False, None)
