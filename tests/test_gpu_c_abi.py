"""GPU tests that call the C ABI of libmi_ns.so directly (ctypes, raw pointers) or need to know which kernel variant
served a shape: the stand-alone Frobenius normalisation, the tile variants of GEMM+AXPY and SYRK, and the
lower-triangle-only output of the direct-to-LDS SYRK kernels.

Bar: bit-exact wherever the arithmetic is exact (integer inputs: sums of squares, products and the correctly rounded
square root and divide are then the same numbers on both sides); float32 round-off otherwise, stated at the assert.
"""

import ctypes

import numpy as np
import pytest
import torch

from emerging_optimizers import _hip, hip_kernels, triton_kernels
from oracle import ns_oracle as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _vp(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _frob(x, *, eps=1e-15, f64=False, out_bf16=False, want_norm=True):
    """mi_frob_normalize on a (batch, rows, cols) float32 tensor; returns (out, dev_norm)."""
    lib = _hip.lib()
    batch, numel = x.shape[0], x[0].numel()
    out = torch.full(x.shape, float("nan"), device=x.device, dtype=BF if out_bf16 else torch.float32)
    partials = torch.empty(lib.mi_frob_partials_len(batch, numel), device=x.device, dtype=torch.float64)
    norm = torch.full((batch,), float("nan"), device=x.device) if want_norm else None
    rc = lib.mi_frob_normalize(_vp(x), batch, numel, eps, int(f64), _vp(out), int(out_bf16), _vp(partials), _vp(norm),
                               _hip.current_stream_ptr(x.device))
    _hip.check(rc)
    torch.cuda.synchronize()
    return out, norm


@pytest.mark.parametrize("shape", [(3, 256, 512), (1, 8, 8), (2, 1000, 1048), (1, 4096, 1024)])
@pytest.mark.parametrize("f64", [False, True])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_frob_normalize_integer_inputs_bit_exact(gpu, shape, f64, out_bf16):
    """Integer entries: the sum of squares is exact in float32 whatever the order, square root and divide are
    correctly rounded on both sides, so float32 output equals the oracle bit for bit and bf16 output its rounding."""
    x = torch.randint(-2, 3, shape, generator=torch.Generator().manual_seed(5)).float()
    assert float((x.double() ** 2).sum(dim=(-2, -1)).max()) < 2**24
    got, norm = _frob(x.to(gpu), f64=f64, out_bf16=out_bf16)
    want = O.frobenius_normalize(x.numpy(), 1e-15, in_double=f64)
    if out_bf16:
        want = O.round_to_bf16(want)
    assert np.array_equal(got.float().cpu().numpy(), want)
    sumsq = (x.numpy().astype(np.float64) ** 2).sum(axis=(-2, -1))
    want_norm = np.sqrt(sumsq).astype(np.float32) if f64 else np.sqrt(sumsq.astype(np.float32))
    assert np.array_equal(norm.cpu().numpy(), want_norm)


@pytest.mark.parametrize("f64", [False, True])
def test_frob_normalize_random_inputs(gpu, f64):
    x = torch.randn(3, 384, 640, generator=torch.Generator().manual_seed(6)) * torch.tensor([1e-3, 1.0, 50.0])[:, None, None]
    got, norm = _frob(x.to(gpu), f64=f64)
    want = O.frobenius_normalize(x.numpy(), 1e-15, in_double=f64)
    # the float32 sums of squares differ by their summation order, the quotients then by a few ulp
    # (the reference's own tolerance for this step is rtol 1e-6, tests/test_muon_utils.py:124-131)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-6, atol=0)
    np.testing.assert_allclose(norm.cpu().numpy(), np.linalg.norm(x.numpy().astype(np.float64), axis=(-2, -1)), rtol=5e-7)
    ref = torch.nn.functional.normalize(x.to(gpu), p=2, dim=(-2, -1), eps=1e-15)
    torch.testing.assert_close(got, ref, rtol=1e-6, atol=0)
    got16, _ = _frob(x.to(gpu), f64=f64, out_bf16=True, want_norm=False)
    want16 = O.round_to_bf16(want)
    mism = np.mean(got16.float().cpu().numpy() != want16)
    assert mism < 1e-3  # an ulp of float32 flips a bf16 rounding on a tiny fraction of entries
    np.testing.assert_allclose(got16.float().cpu().numpy(), want16, rtol=2**-7, atol=0)


def test_frob_normalize_python_wrapper(gpu):
    """hip_kernels.frob_normalize against torch.nn.functional.normalize over the flattened matrix (what the
    reference's driver calls, muon_utils.py:219-222) and against the numpy oracle; batch of 3, both output types,
    float64 accumulation, the divisor handed back."""
    g = torch.Generator(device=gpu).manual_seed(11)
    x = torch.randn(3, 256, 520, device=gpu, generator=g) * torch.tensor([1e-3, 1.0, 40.0], device=gpu)[:, None, None]
    want = torch.nn.functional.normalize(x.flatten(1), p=2, dim=-1, eps=1e-7).view_as(x)
    got, norm = hip_kernels.frob_normalize(x, return_norm=True)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=0)
    torch.testing.assert_close(norm, x.flatten(1).norm(dim=-1), rtol=1e-6, atol=0)
    got64 = hip_kernels.frob_normalize(x, normalize_in_double=True)
    want64 = (x.double() / x.double().flatten(1).norm(dim=-1)[:, None, None]).float()
    torch.testing.assert_close(got64, want64, rtol=2e-7, atol=0)
    assert np.allclose(got64[1].cpu().numpy(), O.frobenius_normalize(x[1].cpu().numpy(), eps=1e-7, in_double=True), rtol=3e-7, atol=0)
    bf = hip_kernels.frob_normalize(x, out_dtype=BF)
    assert bf.dtype == BF and torch.equal(bf, got.to(BF))
    with pytest.raises(RuntimeError):
        hip_kernels.frob_normalize(x.cpu())
    with pytest.raises(ValueError):
        hip_kernels.frob_normalize(x, out_dtype=torch.float16)


def test_frob_normalize_clamp_and_underflow(gpu):
    # all-zero matrix: divisor is eps, result 0, no NaN; dev_norm reports the clamp
    z = torch.zeros(2, 64, 64, device=gpu)
    out, norm = _frob(z, eps=1e-15)
    assert torch.equal(out, z) and torch.equal(norm, torch.full((2,), 1e-15, device=gpu))
    # float32 squares underflow to zero: the float32 norm is the clamp, the float64 norm is not
    tiny = (torch.randn(1, 256, 256, generator=torch.Generator().manual_seed(7)) * 1e-30).to(gpu)
    out32, n32 = _frob(tiny, eps=1e-15)
    assert float(n32[0]) == np.float32(1e-15)
    torch.testing.assert_close(out32, tiny / 1e-15, rtol=1e-6, atol=0)
    out64, n64 = _frob(tiny, f64=True)
    want = O.frobenius_normalize(tiny.cpu().numpy(), in_double=True)
    np.testing.assert_allclose(out64.cpu().numpy(), want, rtol=1e-6, atol=0)
    assert abs(float(out64.double().norm()) - 1.0) < 1e-5
    # dev_norm is optional
    out_b, none = _frob(tiny, f64=True, want_norm=False)
    assert none is None and torch.equal(out_b, out64)


# ---------------------------------------------------------------- which kernel variant served a shape
def rel_fro_t(a, b):
    return float((a - b).norm() / b.norm())


def _int_bf16(shape, lo, hi, dev, seed=0):
    return torch.randint(lo, hi, shape, generator=torch.Generator().manual_seed(seed)).to(BF).to(dev)


# (shape, expected tile rows, tile columns); all on the direct-to-LDS kernel
GEMM_VARIANTS = [
    ((1, 1024, 2304), 256, 128),   # too few 256 x 256 tiles for the chip: 256 x 128 tiles throughout
    ((1, 2048, 4096), 256, 128),
    ((1, 2048, 8192), 256, 256),   # exactly one round of 256 x 256 tiles
    ((2, 128, 512), 128, 256),     # per-head shapes: 128 x 256 tiles
    ((3, 384, 768), 128, 256),
]


@pytest.mark.parametrize("shape,tile_m,tile_n", GEMM_VARIANTS)
@pytest.mark.parametrize("out_dtype", [BF, torch.float32])
def test_gemm_axpy_variants_integer_exact(gpu, shape, tile_m, tile_n, out_dtype):
    b, m, n = shape
    x = _int_bf16((b, m, n), -2, 3, gpu, seed=1)
    bm = _int_bf16((b, m, m), -2, 3, gpu, seed=2)
    got = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5, out_dtype=out_dtype, out_scale=2.0 if out_dtype == torch.float32 else 1.0)
    info = _hip.last_launch()
    assert (info["tile_m"], info["tile_n"], info["fast"]) == (tile_m, tile_n, 1), info
    # small integers: every product and partial sum is exact in float32, so torch's float32 matmul is an exact
    # reference; the oracle confirms it on the first matrix
    ref = 0.5 * x.float() + 0.25 * torch.bmm(bm.float(), x.float())
    if out_dtype == torch.float32:
        assert torch.equal(got, 2.0 * ref)
    else:
        assert torch.equal(got, ref.to(BF))
    want = O.gemm_axpy(bm[0].float().cpu().numpy(), x[0].float().cpu().numpy(), 0.25, 0.5, round_bf16=out_dtype == BF)
    scale = 2.0 if out_dtype == torch.float32 else 1.0
    assert np.array_equal(got[0].float().cpu().numpy(), scale * want)


def test_gemm_axpy_tail_split_integer_exact(gpu):
    """4096 x 14336: 896 tiles of 256 x 256 are 3.5 rounds of 256 CUs, so the last eight tile columns run as 256 x 128
    tiles in a second launch (768 + 256 workgroups)."""
    m, n = 4096, 14336
    x = _int_bf16((m, n), -2, 3, gpu, seed=3)
    bm = _int_bf16((m, m), -2, 3, gpu, seed=4)
    ref = 0.5 * x.float() + 0.25 * (bm.float() @ x.float())
    for out_dtype in (BF, torch.float32):
        got = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5, out_dtype=out_dtype)
        info = _hip.last_launch()
        if torch.cuda.get_device_properties(0).multi_processor_count == 256:
            assert (info["tiles"], info["tile_m"], info["tile_n"]) == (768 + 256, 256, 128), info
        assert torch.equal(got, ref.to(out_dtype))


def test_gemm_axpy_batched_tail_split_integer_exact(gpu):
    """8 x (1792 x 4096): 896 tiles of 256 x 256 are 3.5 rounds of 256 CUs; the last tile row of every matrix runs as
    256 x 128 tiles in a second launch (96 + 32 workgroups per matrix)."""
    b, m, n = 8, 1792, 4096
    x = _int_bf16((b, m, n), -2, 3, gpu, seed=5)
    bm = _int_bf16((b, m, m), -2, 3, gpu, seed=6)
    ref = 0.5 * x.float() + 0.25 * torch.bmm(bm.float(), x.float())
    for out_dtype in (BF, torch.float32):
        got = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5, out_dtype=out_dtype)
        info = _hip.last_launch()
        if torch.cuda.get_device_properties(0).multi_processor_count == 256:
            assert (info["tiles"], info["tile_m"], info["tile_n"]) == (96 + 32, 256, 128), info
        assert torch.equal(got, ref.to(out_dtype))
    want = O.gemm_axpy(bm[7].float().cpu().numpy(), x[7].float().cpu().numpy(), 0.25, 0.5)
    got = hip_kernels.gemm_axpy(bm, x, alpha=0.25, beta=0.5)
    assert np.array_equal(got[7].float().cpu().numpy(), want)


# n, k, transposed operand, expected tile
SYRK_VARIANTS = [
    (1024, 512, False, 128), (1024, 512, True, 128), (1280, 192, True, 128), (4096, 1024, False, 192),
    (2048, 2048, True, 128), (1792, 256, False, 128), (1096, 128, False, 192), (1096, 128, True, 256),
    (512, 256, False, 128), (768, 1024, True, 128), (384, 128, False, 128), (256, 2048, False, 128),  # small matrices of whole 128-row tiles
]


@pytest.mark.parametrize("n,k,trans,tile", SYRK_VARIANTS)
def test_syrk_variants_integer_exact(gpu, mi_option, n, k, trans, tile):
    """Both operand layouts on the direct-to-LDS kernels (a transposed operand has 128- and 256-row tiles and no
    variant for tiles that overhang the matrix: 1096 rows go to the general kernel there)."""
    mi_option("syrk_transpose", 0)  # the K-strided kernels themselves, not the transposing copy
    mi_option("streamk", 0)
    a = _int_bf16((k, n) if trans else (n, k), -3, 3, gpu, seed=n + k)
    if trans:
        a = a.T
    d = triton_kernels.tsyrk_ex(a)
    info = _hip.last_launch()
    assert info["tile_m"] == tile and info["fast"] == (0 if (trans and n % 128) else 1), info
    ref = (a.float() @ a.float().T).to(BF)
    assert torch.equal(d, ref) and torch.equal(d, d.T)
    s = _int_bf16((n, n), -3, 3, gpu, seed=n)
    s = s + s.T
    arg = s.T if trans else s
    d2 = triton_kernels.tsyrk_ex(arg, arg, alpha=0.25, beta=0.25)
    assert torch.equal(d2, torch.addmm(s.float(), s.float(), s.float(), alpha=0.25, beta=0.25).to(BF))
    if n <= 1280:
        assert np.array_equal(d.float().cpu().numpy(), O.syrk(a.float().cpu().numpy()))


@pytest.mark.parametrize("n,k,batch", [(1024, 256, 1), (1280, 128, 2), (1096, 64, 1), (2048, 512, 1), (512, 128, 2)])
@pytest.mark.parametrize("trans", [False, True])
def test_syrk_lower_triangle_only(gpu, n, k, batch, trans):
    """skip_upper_triangle: the diagonal and everything below it are stored; an element above the diagonal is either
    left untouched (NaN here) or holds its correct value."""
    a = _int_bf16((batch, k, n) if trans else (batch, n, k), -3, 3, gpu, seed=n)
    if trans:
        a = a.mT
    out = torch.full((batch, n, n), float("nan"), device=gpu, dtype=BF)
    triton_kernels.batched_tsyrk_ex(a, skip_upper_triangle=True, out=out)
    ref = torch.bmm(a.float(), a.float().mT).to(BF)
    low = torch.tril(torch.ones(n, n, dtype=torch.bool, device=gpu))
    assert torch.equal(out[:, low], ref[:, low])
    up = out[:, ~low]
    assert bool((torch.isnan(up) | (up == ref[:, ~low])).all())
    # with an addend as well (the epilogue's second code path)
    s = _int_bf16((batch, n, n), -3, 3, gpu, seed=n + 1)
    s = s + s.mT
    out2 = torch.full((batch, n, n), float("nan"), device=gpu, dtype=BF)
    triton_kernels.batched_tsyrk_ex(a, s, alpha=0.5, beta=0.25, skip_upper_triangle=True, out=out2)
    ref2 = torch.baddbmm(s.float(), a.float(), a.float().mT, alpha=0.5, beta=0.25).to(BF)
    assert torch.equal(out2[:, low], ref2[:, low])
    up2 = out2[:, ~low]
    assert bool((torch.isnan(up2) | (up2 == ref2[:, ~low])).all())


# ---------------------------------------------------------------- split-tail (stream-K) launch of the lower-triangle kernel
@pytest.mark.parametrize("batch,n,k", [(16, 2048, 8192), (1, 1024, 8192), (3, 1280, 1024), (2, 1536, 4096), (5, 1024, 448),
                                       (30, 1024, 128), (26, 1024, 256)])
def test_syrk_stream_k_integer_exact(gpu, mi_option, batch, n, k):
    """Whole rounds of 256 x 256 tiles, then the left-over tiles with their K range split between workgroups that
    park float32 accumulators in the workspace, then a launch that adds them and writes those tiles.  Small integers
    make every float32 sum exact, so the result must equal the ordinary launch bit for bit.  30 x 1024 x 128: 300
    tiles, 44 left over, 2 K tiles each (the split is capped by K); 26 x 1024 x 256: 260 tiles, 4 left over, 4 K tiles."""
    mi_option("streamk", 1)
    a = _int_bf16((batch, n, k), -2, 3, gpu, seed=n + k)
    print(f"stream-K {batch}x{n}x{k}", flush=True)
    d = triton_kernels.batched_tsyrk_ex(a)
    info = _hip.last_launch()
    assert info["fast"] == 2 and info["tile_m"] == 256, info
    ref = torch.bmm(a.float(), a.float().mT)
    assert torch.equal(d, ref.to(BF)) and torch.equal(d, d.mT)
    s = _int_bf16((batch, n, n), -3, 3, gpu, seed=n)
    s = s + s.mT
    d2 = triton_kernels.batched_tsyrk_ex(a, s, alpha=0.25, beta=0.5)
    assert _hip.last_launch()["fast"] == 2
    assert torch.equal(d2, torch.baddbmm(s.float(), a.float(), a.float().mT, alpha=0.25, beta=0.5).to(BF))
    mi_option("streamk", 0)
    d3 = triton_kernels.batched_tsyrk_ex(a)
    assert _hip.last_launch()["fast"] == 1 and torch.equal(d3, d)
    if batch * n <= 1280:
        assert np.array_equal(d[0].float().cpu().numpy(), O.syrk(a[0].float().cpu().numpy()))


def test_syrk_stream_k_random_inputs_and_model_choice(gpu, mi_option):
    """Gaussian operands: the stream-K launch adds the same products in another order (float32), so it agrees with the
    ordinary launch to bf16 rounding of near-ties; which launch the cost model picks for the benchmark shapes."""
    mi_option("streamk", -1)
    a = torch.randn(16, 2048, 8192, device=gpu, generator=torch.Generator(device=gpu).manual_seed(5)).to(BF)
    d = triton_kernels.batched_tsyrk_ex(a)
    chosen = _hip.last_launch()
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert chosen["fast"] == 2, chosen  # 576 tiles of 256 x 256 = 2.25 rounds of 256 CUs
    mi_option("streamk", 0)
    d0 = triton_kernels.batched_tsyrk_ex(a)
    assert _hip.last_launch()["fast"] == 1
    diff = (d.float() - d0.float()).abs()
    # one bf16 ulp at most, and only where the float32 sums straddle a rounding boundary
    assert float((diff / d0.float().abs().clamp_min(1.0)).max()) <= 2.0 ** -7
    assert float((diff > 0).float().mean()) < 0.02
    ref = a[3].float() @ a[3].float().T
    assert rel_fro_t(d[3].float(), ref) < 3e-3
    mi_option("streamk", -1)
    x = torch.randn(4096, 14336, device=gpu).to(BF)
    triton_kernels.tsyrk_ex(x)
    assert _hip.last_launch()["fast"] == 1  # 253 tiles of 192 x 192: one round already


# ---------------------------------------------------------------- K-strided operand through a transposed copy
@pytest.mark.parametrize("batch,n,k", [(1, 1024, 512), (2, 1096, 192), (1, 4096, 14336), (3, 1280, 4096), (16, 2048, 8192)])
def test_syrk_transposed_copy_integer_exact(gpu, mi_option, batch, n, k):
    """A K-strided operand is first copied, transposed, into the workspace and then multiplied by the K-contiguous
    kernels (which have a 192 x 192 tile and the faster K loop).  Bit-equal to the K-strided kernels on small integers.
    4096 x 14336 is a shape where the model itself chooses the copy (elsewhere it is forced here); 16 x 2048 x 8192
    adds the split-tail launch behind it, both parts of the workspace in use."""
    forced = (n, k) != (4096, 14336)
    if forced:
        mi_option("syrk_transpose", 1)
    else:
        mi_option("syrk_transpose", -1)
    a = _int_bf16((batch, k, n), -2, 3, gpu, seed=n + k + 1).mT  # stored as k rows of n
    assert a.stride(-2) == 1
    print(f"transposed copy {batch}x{n}x{k}", flush=True)
    lib = _hip.lib()
    need = lib.mi_syrk_workspace_bytes(batch, n, k, 1)
    assert need >= batch * n * k * 2
    d = triton_kernels.batched_tsyrk_ex(a)
    info = _hip.last_launch()
    if k % 64 == 0 and n >= 1024:
        assert info["fast"] in (1, 2) and (info["tile_m"] == 192 if (n, k) == (4096, 14336) else True), info
    ref = torch.bmm(a.float(), a.float().mT).to(BF)
    assert torch.equal(d, ref)
    s = _int_bf16((batch, n, n), -3, 3, gpu, seed=n)
    s = s + s.mT
    d2 = triton_kernels.batched_tsyrk_ex(a, s, alpha=0.25, beta=0.5)
    assert torch.equal(d2, torch.baddbmm(s.float(), a.float(), a.float().mT, alpha=0.25, beta=0.5).to(BF))
    mi_option("syrk_transpose", 0)
    assert torch.equal(triton_kernels.batched_tsyrk_ex(a), d)
    assert lib.mi_syrk_workspace_bytes(batch, n, k, 1) < batch * n * k * 2
