"""The allocation-free Newton-Schulz entry point (``mi_newton_schulz_bf16_noalloc``: workspace inside the library)
against ``mi_newton_schulz_bf16`` with a caller-provided workspace, both called through the C ABI.  The two run the
same kernels on the same layout, so their results must agree bit for bit -- also on a second call with a smaller
input, which finds the previous call's contents in the shared buffer.
"""

import ctypes

import pytest
import torch

from emerging_optimizers import _hip

pytestmark = pytest.mark.gpu
QUINTIC = [(4.0848, -6.8946, 2.9270), (3.9505, -6.3029, 2.6377), (3.7418, -5.5913, 2.3037), (2.8769, -3.1427, 1.2046),
           (2.8366, -3.0525, 1.2012)]


def _vp(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(x, steps=5, out_scale=1.0):
    lib = _hip.lib()
    batch = x.shape[0] if x.dim() == 3 else 1
    rows, cols = x.shape[-2:]
    flat = [v for abc in QUINTIC[:steps] for v in abc]
    abc = (ctypes.c_float * max(len(flat), 1))(*flat)
    stream = _hip.current_stream_ptr(x.device)
    nbytes = lib.mi_newton_schulz_workspace_bytes(batch, rows, cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    want = torch.full_like(x, float("nan"))
    _hip.check(lib.mi_newton_schulz_bf16(_vp(x), _vp(want), batch, rows, cols, abc, steps, 1e-15, 0, out_scale, _vp(ws), nbytes, stream))
    got = torch.full_like(x, float("nan"))
    # A first call looks up the buffer's address (once per device) and makes the runtime load the code of the kernels
    # this shape uses; the call that is measured comes after it.  Free device memory as the driver reports it
    # (hipMemGetInfo) sees every allocation of the process, torch's own and any the library might make.
    _hip.check(lib.mi_newton_schulz_bf16_noalloc(_vp(x), _vp(got), batch, rows, cols, abc, steps, 1e-15, 0, out_scale, stream))
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(x.device)[0]
    torch_before = torch.cuda.memory_allocated(x.device)
    rc = lib.mi_newton_schulz_bf16_noalloc(_vp(x), _vp(got), batch, rows, cols, abc, steps, 1e-15, 0, out_scale, stream)
    _hip.check(rc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(x.device)[0] == free_before
    assert torch.cuda.memory_allocated(x.device) == torch_before
    return got, want


def test_noalloc_entry_matches_the_workspace_entry_on_consecutive_calls(gpu):
    gen = torch.Generator().manual_seed(21)
    # a wide matrix that takes its steps in groups, then smaller inputs that reuse the same buffer: a batch of
    # per-head shapes (split-K Gram path), a tall matrix (transposing cast, staged result) and a tiny one
    shapes = [(1024, 4096), (4, 128, 1024), (1536, 256), (64, 128), (1024, 4096)]
    first = None
    for shape in shapes:
        x = (torch.randn(*shape, generator=gen) * 1e-2).to(gpu)
        got, want = _both(x)
        assert not torch.isnan(got).any()
        assert torch.equal(got, want), shape
        if first is None:
            first = (x, got)
    # the first input again, after the others have overwritten the buffer
    again, _ = _both(first[0])
    assert torch.equal(again, first[1])
    # steps = 0 (normalisation only) and an output scale
    x = torch.randn(256, 512, generator=gen).to(gpu)
    got, want = _both(x, steps=0, out_scale=3.0)
    assert torch.equal(got, want)
    torch.testing.assert_close(got, 3.0 * x / x.norm(), rtol=1e-6, atol=0)


def test_noalloc_entry_refuses_what_does_not_fit(gpu):
    lib = _hip.lib()
    abc = (ctypes.c_float * 15)(*[v for c in QUINTIC for v in c])
    x = torch.zeros(8, device=gpu)
    assert lib.mi_newton_schulz_workspace_bytes(1, 4096, 14336) > (128 << 20)
    rc = lib.mi_newton_schulz_bf16_noalloc(_vp(x), _vp(x), 1, 4096, 14336, abc, 5, 1e-15, 0, 1.0, None)
    assert rc == _hip.MI_ERR_WORKSPACE and "built-in buffer" in _hip.last_error()
    assert lib.mi_newton_schulz_bf16_noalloc(_vp(x), _vp(x), 1, 12, 16, abc, 5, 1e-15, 0, 1.0, None) == _hip.MI_ERR_UNSUPPORTED_SHAPE
    assert lib.mi_newton_schulz_bf16_noalloc(_vp(x), _vp(x), 0, 16, 16, abc, 5, 1e-15, 0, 1.0, None) == _hip.MI_OK
