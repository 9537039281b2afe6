"""The shared library loads and exports exactly what include/mi_ns.h declares; argument validation that
needs no GPU returns the documented error codes.  No kernel is launched here."""

import ctypes
import os
import re

import pytest
import torch

from emerging_optimizers import _hip, hip_kernels, triton_kernels

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "mi_ns.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared_symbols()
    assert names == sorted(n for n, _, _ in _hip.EXPORTS), "binding table and header disagree"
    lib = _hip.lib()
    for name in names:
        assert getattr(lib, name) is not None


def test_version_and_flags():
    assert _hip.lib().mi_version() >= 100
    assert hip_kernels.HAS_HIP_KERNELS is True and triton_kernels.HAS_TRITON_340 is True
    assert triton_kernels.tsyrk_ex is hip_kernels.tsyrk_ex


def test_validation_codes_without_gpu():
    lib = _hip.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(ctypes.addressof(buf) & ~15, ctypes.c_void_p)
    # N not a multiple of 8
    rc = lib.mi_syrk_bf16(p, 1, 12, 16, 192, 16, 0, None, 0, 12, 1.0, 0.0, p, 144, 12, 0, None)
    assert rc == _hip.MI_ERR_UNSUPPORTED_SHAPE and "multiples of 8" in _hip.last_error()
    # beta != 0 without C
    assert lib.mi_syrk_bf16(p, 1, 16, 16, 256, 16, 0, None, 0, 16, 1.0, 0.5, p, 256, 16, 0, None) == _hip.MI_ERR_BAD_ARG
    assert lib.mi_syrk_bf16(None, 1, 16, 16, 256, 16, 0, None, 0, 16, 1.0, 0.0, p, 256, 16, 0, None) == _hip.MI_ERR_BAD_ARG
    assert lib.mi_gemm_axpy_bf16(p, 0, 12, p, 0, 16, 0, p, 0, 16, 1, 12, 16, 1.0, 1.0, 0, 1.0, None) == _hip.MI_ERR_UNSUPPORTED_SHAPE
    assert lib.mi_frob_normalize(p, 1, 12, 1e-15, 0, p, 1, p, None, None) == _hip.MI_ERR_UNSUPPORTED_SHAPE
    # empty problems are no-ops
    assert lib.mi_syrk_bf16(p, 0, 16, 16, 256, 16, 0, None, 0, 16, 1.0, 0.0, p, 256, 16, 0, None) == _hip.MI_OK
    assert lib.mi_newton_schulz_workspace_bytes(1, 4096, 14336) >= 2 * 4096 * 14336 * 2 + 2 * 4096 * 4096 * 2
    assert lib.mi_newton_schulz_workspace_bytes(0, 8, 8) == 0
    abc = (ctypes.c_float * 3)(1, 2, 3)
    assert lib.mi_newton_schulz_bf16(p, p, 1, 12, 16, abc, 1, 1e-15, 0, 1.0, p, 10**9, None) == _hip.MI_ERR_UNSUPPORTED_SHAPE
    assert lib.mi_newton_schulz_bf16(p, p, 1, 16, 16, abc, 1, 1e-15, 0, 1.0, p, 8, None) == _hip.MI_ERR_WORKSPACE
    assert lib.mi_frob_partials_len(3, 1024) >= 3


def test_python_validation_messages_cpu():
    """Exception types and messages of the SYRK wrappers (test_triton_kernels.py:220-441 of the reference);
    all of these fire before any device work, so they can be checked on CPU tensors."""
    bf = torch.bfloat16
    for fn in (triton_kernels.tsyrk_ex, triton_kernels.tsyrk_ex_small_matrix):
        with pytest.raises(TypeError, match="must be bfloat16"):
            fn(torch.randn(4, 4))
        with pytest.raises(TypeError, match="must be 2D"):
            fn(torch.randn(4).to(bf))
        with pytest.raises(TypeError, match="must be contiguous"):
            fn(torch.randn(8, 8).to(bf)[:, ::2])
        with pytest.raises(RuntimeError, match=r"c must be of shape \(N, N\)"):
            fn(torch.randn(4, 4).to(bf), torch.randn(3, 3).to(bf), beta=1.0)
        with pytest.raises(RuntimeError, match="c or c.T must be contiguous"):
            fn(torch.randn(8, 8).to(bf), torch.randn(16, 16).to(bf)[::2, ::2], beta=1.0)
    with pytest.raises(RuntimeError, match="out must be same shape/device/dtype"):
        triton_kernels.tsyrk_ex_small_matrix(torch.randn(4, 4).to(bf), out=torch.empty(3, 3, dtype=bf))
    with pytest.raises(RuntimeError, match="out must be contiguous"):
        triton_kernels.tsyrk_ex_small_matrix(torch.randn(4, 4).to(bf), out=torch.empty(8, 8, dtype=bf)[::2, ::2])
    b = triton_kernels.batched_tsyrk_ex
    with pytest.raises(TypeError, match="must be bfloat16"):
        b(torch.randn(2, 16, 16))
    with pytest.raises(TypeError, match="must be 3D"):
        b(torch.randn(16, 16).to(bf))
    with pytest.raises(TypeError, match="must be contiguous"):
        b(torch.randn(2, 16, 32).to(bf)[:, :, ::2])
    for shape in [(2, 12, 16), (2, 16, 12)]:
        with pytest.raises(RuntimeError, match="must be multiples of 8"):
            b(torch.randn(*shape).to(bf))
    with pytest.raises(RuntimeError, match=r"c must be of shape \(B, N, N\)"):
        b(torch.randn(2, 16, 16).to(bf), torch.randn(2, 8, 8).to(bf), beta=1.0)
    with pytest.raises(RuntimeError, match="c or c.mT must be contiguous"):
        b(torch.randn(2, 16, 16).to(bf), torch.randn(2, 32, 32).to(bf)[:, ::2, ::2], beta=1.0)
    with pytest.raises(RuntimeError, match="out must be same shape/device/dtype"):
        b(torch.randn(2, 16, 16).to(bf), out=torch.empty(2, 8, 8, dtype=bf))
    with pytest.raises(RuntimeError, match="out must be contiguous"):
        b(torch.randn(2, 16, 16).to(bf), out=torch.empty(2, 32, 32, dtype=bf)[:, ::2, ::2])
    # CPU tensors are refused loudly rather than computed some other way
    with pytest.raises(RuntimeError, match="GPU only"):
        triton_kernels.tsyrk_ex(torch.randn(8, 8).to(bf))
    assert triton_kernels.can_use_batched_tsyrk(torch.randn(2, 16, 16).to(bf)) is False  # not on the GPU


@pytest.mark.parametrize("env", [None, "0", "pairs", "force"])
def test_step_grouping_rule_matches_the_oracle_model(mi_option, env):
    """The host-side rule of the driver (which steps share a Gram matrix) against the oracle's restatement of it,
    over shapes on both sides of every threshold and every coefficient family."""
    from oracle import ns_oracle as O

    mi_option("ns_pairs", {None: -1, "0": 0, "pairs": 1, "force": 2}[env])
    lib = _hip.lib()
    shapes = [(1, 4096, 14336), (1, 14336, 4096), (8, 4096, 14336), (1, 4096, 4096), (1, 4096, 8184), (1, 4096, 8192),
              (1, 1024, 2048), (1, 1016, 4096), (32, 128, 4096), (2, 256, 1536), (4, 128, 1000), (1, 384, 4096), (1, 8, 16)]
    cases = [("simple", 5), ("quintic", 5), ("quintic", 4), ("quintic", 3), ("polar_express", 8), ("cans", 5), ("aol", 5),
             ("deepseekv4", 10), ("cubic5", 5), ("simple", 1), ("simple", 2)]
    for batch, rows, cols in shapes:
        m, n = min(rows, cols), max(rows, cols)
        split_k = m % 128 == 0 and m <= 256 and n % 512 == 0 and n >= 1024 and batch * (n // 512) <= 65535
        rule = 2 if (split_k or (m >= 1024 and n >= 2 * m)) else 0
        mode = {None: rule, "0": 0, "pairs": min(rule, 1), "force": 1}[env]
        for kind, steps in cases:
            coeffs = O.expand_coefficients(steps, kind)
            abc = (ctypes.c_float * (3 * steps))(*[v for c in coeffs for v in c])
            out = (ctypes.c_int * 16)()
            count = lib.mi_newton_schulz_schedule(batch, rows, cols, abc, steps, out, 16)
            assert list(out[:count]) == O.group_schedule(coeffs, mode), (env, batch, rows, cols, kind, steps)
    assert lib.mi_newton_schulz_schedule(1, 64, 64, None, 5, (ctypes.c_int * 4)(), 4) == _hip.MI_ERR_BAD_ARG


def test_options_are_set_once_and_read_back(mi_option):
    """mi_set_option / mi_get_option: ranges, unknown names, and that the step-grouping option steers both the
    schedule query and the workspace size (two more m x m buffers where steps share a Gram matrix)."""
    lib = _hip.lib()
    assert _hip.get_option("ns_pairs") == -1 and _hip.get_option("streamk") == -1 and _hip.get_option("tall_direct") == 1
    assert lib.mi_set_option(b"no_such_option", 1) == _hip.MI_ERR_BAD_ARG and "unknown option" in _hip.last_error()
    assert lib.mi_set_option(b"ns_pairs", 3) == _hip.MI_ERR_BAD_ARG and "-1 .. 2" in _hip.last_error()
    assert lib.mi_set_option(b"head_apply", -1) == _hip.MI_ERR_BAD_ARG
    assert lib.mi_get_option(b"ns_pairs", None) == _hip.MI_ERR_BAD_ARG
    assert _hip.get_option("ns_pairs") == -1  # a refused value changes nothing
    grouped = lib.mi_newton_schulz_workspace_bytes(1, 4096, 14336)
    mi_option("ns_pairs", 0)
    assert _hip.get_option("ns_pairs") == 0
    assert grouped - lib.mi_newton_schulz_workspace_bytes(1, 4096, 14336) == 2 * 4096 * 4096 * 2
    # tall inputs whose last product writes the result transposed need no float32 staging copy
    direct = lib.mi_newton_schulz_workspace_bytes(1, 14336, 4096)
    mi_option("tall_direct", 0)
    assert lib.mi_newton_schulz_workspace_bytes(1, 14336, 4096) - direct == 14336 * 4096 * 4


def test_tall_input_beyond_the_fast_loaders_keeps_its_staging_copy():
    """The direct-to-LDS loaders address a tile's rows with 32-bit byte offsets and leave leading dimensions of 4M
    elements and more to the general kernel, which cannot write its result transposed: such a tall input must be given
    the float32 staging copy by the workspace layout (it was once laid out without, and the refusal came after the first
    kernel had run)."""
    lib = _hip.lib()
    rows, cols = (1 << 22) + 1024, 1024
    wide = lib.mi_newton_schulz_workspace_bytes(1, cols, rows)
    tall = lib.mi_newton_schulz_workspace_bytes(1, rows, cols)
    assert tall - wide == rows * cols * 4
    rows = (1 << 22) - 1024  # just inside: written directly, no staging copy
    assert lib.mi_newton_schulz_workspace_bytes(1, rows, cols) == lib.mi_newton_schulz_workspace_bytes(1, cols, rows)


def test_syrk_with_workspace_validates_before_it_copies():
    """mi_syrk_bf16_ws refuses a bad call before its transposing copy of a K-strided operand (nothing is launched: this
    runs without a GPU)."""
    lib = _hip.lib()
    buf = (ctypes.c_char * 8192)()
    p = ctypes.cast((ctypes.addressof(buf) + 255) & ~255, ctypes.c_void_p)
    args = lambda D, c_ld, beta, C: (p, 1, 2048, 4096, 2048 * 4096, 2048, 1, C, 2048 * 2048, c_ld, 1.0, beta, D, 2048 * 2048, 2048, 0,
                                     p, 1 << 40, None)
    assert lib.mi_syrk_bf16_ws(*args(None, 2048, 0.0, None)) == _hip.MI_ERR_BAD_ARG  # D missing
    assert lib.mi_syrk_bf16_ws(*args(p, 2048, 0.5, None)) == _hip.MI_ERR_BAD_ARG     # beta without C
    assert lib.mi_syrk_bf16_ws(*args(p, 2044, 0.5, p)) == _hip.MI_ERR_UNSUPPORTED_SHAPE  # c_ld not a multiple of 8
    assert lib.mi_syrk_bf16_ws(*args(p, 1024, 0.5, p)) == _hip.MI_ERR_BAD_ARG        # c_ld too small
