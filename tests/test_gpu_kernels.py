"""GPU parity tests of the SYRK and GEMM+AXPY kernels, called through the package (ctypes -> C ABI).

Bar: bit-exact against the numpy oracle wherever the arithmetic is exact (integer inputs, power-of-two
scalars -- the reference's own exactness device, tests/test_triton_kernels.py:293-363, 444-480 there);
rtol 0.05 on random inputs as in the reference; bitwise symmetry everywhere.
"""

import numpy as np
import pytest
import torch

from emerging_optimizers import hip_kernels, triton_kernels
from oracle import ns_oracle as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _np(t):
    return t.float().cpu().numpy()


def _int_bf16(shape, lo, hi, dev):
    return torch.randint(lo, hi, shape, device=dev).to(BF)


SYRK_2D = [triton_kernels.tsyrk_ex, triton_kernels.tsyrk_ex_small_matrix]


@pytest.mark.parametrize("fn", SYRK_2D)
@pytest.mark.parametrize("n,k", [(128, 128), (256, 64), (64, 64), (16, 128), (8, 8), (264, 72), (1024, 512), (1280, 192)])
@pytest.mark.parametrize("trans", [False, True])
def test_syrk_integer_exact(gpu, fn, n, k, trans):
    a = _int_bf16((k, n) if trans else (n, k), -3, 3, gpu)
    if trans:
        a = a.T
    d = fn(a)  # no warm-up call: the first launch must already be right
    assert np.array_equal(_np(d), O.syrk(_np(a)))
    assert torch.equal(d, (a.float() @ a.float().T).to(BF))
    assert torch.equal(d, d.T)


@pytest.mark.parametrize("fn", SYRK_2D)
@pytest.mark.parametrize("n,alpha", [(128, 0.5), (256, 0.25), (1024, 0.25), (5120, 0.25)])  # 5120: 256 x 256 tiles
@pytest.mark.parametrize("trans", [False, True])
def test_syrk_addmm_integer_exact(gpu, fn, n, alpha, trans):
    s = _int_bf16((n, n), -3, 3, gpu)
    s = s + s.T
    arg = s.T if trans else s
    d = fn(arg, arg, alpha=alpha, beta=alpha)
    assert np.array_equal(_np(d), O.syrk(_np(s), _np(s), alpha, alpha))
    assert torch.equal(d, torch.addmm(s.float(), s.float(), s.float(), alpha=alpha, beta=alpha).to(BF))


@pytest.mark.parametrize("fn", SYRK_2D)
@pytest.mark.parametrize("n,k,atol", [(128, 128, 0.0), (256, 64, 0.1)])
@pytest.mark.parametrize("trans", [False, True])
def test_syrk_random_close_to_matmul(gpu, fn, n, k, atol, trans):
    a = torch.randn(n, k, device=gpu, dtype=BF)
    if trans:
        a = a.T.contiguous().T
    torch.testing.assert_close(fn(a), a @ a.T, atol=atol, rtol=0.05)
    sym = torch.randn(n, n, device=gpu, dtype=BF)
    sym = sym + sym.T
    torch.testing.assert_close(fn(sym, sym, alpha=0.4, beta=0.3), torch.addmm(sym, sym, sym, alpha=0.4, beta=0.3), atol=0, rtol=0.05)


def test_syrk_out_argument_and_poison(gpu):
    a = torch.randn(256, 64, device=gpu, dtype=BF)
    out = torch.full((256, 256), float("nan"), device=gpu, dtype=BF)
    res = triton_kernels.tsyrk_ex_small_matrix(a, out=out)
    assert res is out and not torch.isnan(out).any()  # every element of both triangles was written
    assert torch.equal(out, triton_kernels.tsyrk_ex_small_matrix(a))
    b = torch.randn(3, 1280, 128, device=gpu, dtype=BF)
    outb = torch.full((3, 1280, 1280), float("nan"), device=gpu, dtype=BF)
    triton_kernels.batched_tsyrk_ex(b, out=outb)
    assert not torch.isnan(outb).any() and torch.equal(outb, outb.mT)


def test_syrk_skip_upper_triangle(gpu):
    a = _int_bf16((2, 512, 128), -3, 3, gpu)
    d = triton_kernels.batched_tsyrk_ex(a, skip_upper_triangle=True)
    ref = torch.bmm(a.float(), a.float().mT).to(BF)
    assert torch.equal(torch.tril(d.float()), torch.tril(ref.float()))


# (8, 1024, 256): 128 x 128 tiles two to a CU; (8, 1792, 4096): 256 x 256 tiles, then 128 x 128 with addend;
# (4, 2048, 2048): 544 tiles of 128 x 128, more than one round of two per CU
@pytest.mark.parametrize("b,n,k", [(2, 128, 128), (4, 256, 64), (8, 16, 128), (2, 1024, 64), (3, 40, 24), (8, 1024, 256), (8, 1792, 4096),
                                   (4, 2048, 2048)])
@pytest.mark.parametrize("trans", [False, True])
def test_batched_syrk_integer_exact(gpu, b, n, k, trans):
    a = _int_bf16((b, k, n) if trans else (b, n, k), -3, 3, gpu)
    if trans:
        a = a.mT
    d = triton_kernels.batched_tsyrk_ex(a)
    assert np.array_equal(_np(d), O.syrk(_np(a)))
    assert torch.equal(d, torch.bmm(a.float(), a.float().mT).to(BF)) and torch.equal(d, d.mT)
    s = _int_bf16((b, n, n), -3, 3, gpu)
    s = s + s.mT
    arg = s.mT if trans else s
    for alpha in (0.5, 0.25):
        d = triton_kernels.batched_tsyrk_ex(arg, arg, alpha=alpha, beta=alpha)
        assert np.array_equal(_np(d), O.syrk(_np(s), _np(s), alpha, alpha))


def test_batched_equals_loop_of_2d(gpu):
    a = torch.randn(5, 384, 256, device=gpu, dtype=BF)
    batched = triton_kernels.batched_tsyrk_ex(a)
    assert torch.equal(batched, torch.stack([triton_kernels.tsyrk_ex(a[i]) for i in range(5)]))


def test_can_use_batched_tsyrk_truth_table(gpu):
    a = torch.randn(2, 128, 64, device=gpu, dtype=BF)
    c = torch.randn(2, 128, 128, device=gpu, dtype=BF)
    r = lambda *s: torch.randn(*s, device=gpu, dtype=BF)
    cases = [
        (a, None, True), (r(2, 64, 128).mT, None, True), (a, c, True), (a.float(), None, False), (a[0], None, False),
        (r(2, 12, 64), None, False), (r(2, 128, 12), None, False), (c[:, :, ::2], None, False),
        (a, r(2, 64, 64), False), (a, c.float(), False), (a, r(2, 256, 256)[:, ::2, ::2], False),
    ]
    for x, y, want in cases:
        assert triton_kernels.can_use_batched_tsyrk(x, y) is want


def test_syrk_config2_shape_properties(gpu):
    """Batch 16 of 2048 x 8192, entries N(0, 0.02^2): bitwise symmetry, agreement with a float32 bmm, and
    linearity in alpha -- properties that do not need a CPU reference at this size."""
    g = torch.Generator(device="cpu").manual_seed(0)
    a = (torch.randn(16, 2048, 8192, generator=g) * 0.02).to(BF).to(gpu)
    d = triton_kernels.batched_tsyrk_ex(a)
    assert torch.equal(d, d.mT)
    ref = torch.bmm(a.float(), a.float().mT)
    assert float((d.float() - ref).norm() / ref.norm()) < 3e-3  # one bf16 rounding: ~2^-9 / sqrt(3)
    assert (d.float() - ref).abs().max() <= ref.abs().max() * 2**-8
    d2 = triton_kernels.batched_tsyrk_ex(a, alpha=2.0)
    assert torch.equal(d2.float(), 2.0 * d.float())  # scaling by a power of two commutes with rounding
    # sub-block oracle check on CPU (first matrix, first 256 rows)
    sub = O.syrk(_np(a[0, :256]))
    mism = np.mean(_np(d[0, :256, :256]) != sub)
    assert mism < 2e-3  # summation order may flip a rounding on a tiny fraction of entries


# ---------------------------------------------------------------- GEMM + AXPY
@pytest.mark.parametrize("b,m,n", [(1, 32, 64), (2, 128, 256), (1, 256, 1024), (1, 1024, 2304), (1, 1024, 16640), (3, 64, 8), (1, 8, 64), (2, 264, 520),
                                   (2, 128, 512), (3, 384, 768), (1, 512, 256), (5, 896, 256)])
@pytest.mark.parametrize("trans", [False, True])
def test_gemm_axpy_integer_exact(gpu, b, m, n, trans):
    x = _int_bf16((b, n, m) if trans else (b, m, n), -2, 3, gpu)
    if trans:
        x = x.mT
    bm = _int_bf16((b, m, m), -2, 3, gpu)  # not symmetric on purpose
    got = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5)
    want = O.gemm_axpy(_np(bm), _np(x), 0.25, 0.5)
    assert got.shape == x.shape and got.stride() == x.stride()
    assert np.array_equal(_np(got), want)
    got32 = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5, out_dtype=torch.float32, out_scale=2.0)
    assert np.array_equal(got32.cpu().numpy(), 2.0 * O.gemm_axpy(_np(bm), _np(x), 0.25, 0.5, round_bf16=False))
    if b == 1:
        got2d = hip_kernels.gemm_axpy(bm[0], x[0], alpha=0.25, beta=0.5)
        assert torch.equal(got2d, got[0])


def test_gemm_axpy_random_close_to_addmm(gpu):
    x = torch.randn(1024, 4096, device=gpu, dtype=BF) * 0.05
    bm = torch.randn(1024, 1024, device=gpu, dtype=BF) * 0.05
    got = hip_kernels.gemm_axpy(bm, x, alpha=1.0, beta=3.4445)
    ref = 3.4445 * x.float() + bm.float() @ x.float()
    assert float((got.float() - ref).norm() / ref.norm()) < 3e-3
    gott = hip_kernels.gemm_axpy(bm, x.T.contiguous().T, alpha=1.0, beta=3.4445)
    assert torch.equal(gott, got)  # both memory layouts accumulate in the same k order


def test_gemm_axpy_errors(gpu):
    x = torch.randn(16, 32, device=gpu, dtype=BF)
    with pytest.raises(TypeError, match="bfloat16"):
        hip_kernels.gemm_axpy(x.float()[:, :16], x)
    with pytest.raises(RuntimeError, match="shape"):
        hip_kernels.gemm_axpy(torch.zeros(8, 8, device=gpu, dtype=BF), x)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        hip_kernels.gemm_axpy(torch.zeros(12, 12, device=gpu, dtype=BF), torch.zeros(12, 16, device=gpu, dtype=BF))
