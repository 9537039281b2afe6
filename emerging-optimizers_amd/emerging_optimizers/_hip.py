"""ctypes binding of ``libmi_ns.so`` (the gfx950 HIP kernels behind this package).

The shared library is built in-tree by ``csrc/Makefile`` (``__graft_entry__.build()`` drives it).
There is deliberately no software fallback for device tensors: every wrapper below raises
``RuntimeError`` if the library cannot be loaded, so a missing build can never be mistaken for a
working accelerated path.
"""

from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

import torch


_LIB_NAME = "libmi_ns.so"
_CSRC_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_PATH = os.path.join(_CSRC_DIR, _LIB_NAME)

MI_OK = 0
MI_ERR_BAD_ARG = -1
MI_ERR_UNSUPPORTED_SHAPE = -2
MI_ERR_LAUNCH = -3
MI_ERR_WORKSPACE = -4

# Every symbol include/mi_ns.h declares: (name, restype, argtypes)
_i64, _int, _f32, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
EXPORTS = (
    ("mi_version", _int, ()),
    ("mi_last_error", ctypes.c_char_p, ()),
    ("mi_syrk_bf16", _int, (_vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _i64, _f32, _f32, _vp, _i64, _i64, _int, _vp)),
    ("mi_syrk_workspace_bytes", _sz, (_i64, _i64, _i64, _int)),
    (
        "mi_syrk_bf16_ws",
        _int,
        (_vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _i64, _f32, _f32, _vp, _i64, _i64, _int, _vp, _sz, _vp),
    ),
    (
        "mi_gemm_axpy_bf16",
        _int,
        (_vp, _i64, _i64, _vp, _i64, _i64, _int, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _int, _f32, _vp),
    ),
    ("mi_frob_normalize", _int, (_vp, _i64, _i64, _f32, _int, _vp, _int, _vp, _vp, _vp)),
    ("mi_frob_partials_len", _sz, (_i64, _i64)),
    ("mi_newton_schulz_bf16", _int, (_vp, _vp, _i64, _i64, _i64, _vp, _int, _f32, _int, _f32, _vp, _sz, _vp)),
    ("mi_newton_schulz_workspace_bytes", _sz, (_i64, _i64, _i64)),
    ("mi_newton_schulz_bf16_noalloc", _int, (_vp, _vp, _i64, _i64, _i64, _vp, _int, _f32, _int, _f32, _vp)),
    ("mi_newton_schulz_schedule", _int, (_i64, _i64, _i64, _vp, _int, _vp, _int)),
    (
        "mi_muon_update_bf16",
        _int,
        (_vp, _vp, _vp, _i64, _i64, _i64, _f32, _int, _f32, _f32, _vp, _int, _f32, _int, _vp, _sz, _vp),
    ),
    ("mi_profile_begin", _int, ()),
    ("mi_profile_end", _int, (_vp, _vp)),
    ("mi_debug_last_launch", _int, (_vp, _vp, _vp, _vp)),
    ("mi_set_option", _int, (ctypes.c_char_p, _int)),
    ("mi_get_option", _int, (ctypes.c_char_p, _vp)),
)

_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_load_error: Optional[str] = None


def _try_load() -> None:
    global _lib, _load_error
    with _lock:
        if _lib is not None or _load_error is not None:
            return
        if not os.path.exists(LIB_PATH):
            _load_error = f"{LIB_PATH} not found; build it with `make -C {_CSRC_DIR}`"
            return
        try:
            lib = ctypes.CDLL(LIB_PATH)
            for name, restype, argtypes in EXPORTS:
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = list(argtypes)
            _lib = lib
        except (OSError, AttributeError) as exc:  # missing ROCm runtime, or a stale build lacking a symbol
            _load_error = f"cannot load {LIB_PATH}: {exc}"


def available() -> bool:
    """True when the HIP library is loadable (says nothing about a GPU being present)."""
    _try_load()
    return _lib is not None


def lib() -> ctypes.CDLL:
    """The loaded library; raises ``RuntimeError`` when it is missing (no fallback)."""
    _try_load()
    if _lib is None:
        raise RuntimeError(f"HIP extension unavailable: {_load_error}")
    return _lib


_gfx950: dict[int, bool] = {}


def device_is_gfx950(device: torch.device) -> bool:
    """Whether ``device`` is the part the kernels are compiled for (cached per device index)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    hit = _gfx950.get(idx)
    if hit is None:
        arch = getattr(torch.cuda.get_device_properties(idx), "gcnArchName", "")
        hit = _gfx950[idx] = arch.startswith("gfx950")
    return hit


def last_launch() -> dict:
    """Tile shape and workgroup count of the last product this thread launched (see ``mi_debug_last_launch``)."""
    vals = [ctypes.c_int(0) for _ in range(4)]
    check(lib().mi_debug_last_launch(*[ctypes.byref(v) for v in vals]))
    return dict(zip(("tiles", "tile_m", "tile_n", "fast"), (v.value for v in vals)))


def set_option(name: str, value: int) -> int:
    """Sets a process-wide option of the library (see ``mi_set_option``); returns the previous value."""
    prev = get_option(name)
    check(lib().mi_set_option(name.encode(), int(value)))
    return prev


def get_option(name: str) -> int:
    out = ctypes.c_int(0)
    check(lib().mi_get_option(name.encode(), ctypes.byref(out)))
    return out.value


def last_error() -> str:
    return lib().mi_last_error().decode("utf-8", "replace")


def current_stream_ptr(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def check(rc: int, unsupported_exc: type = RuntimeError) -> None:
    """Turn a negative MI_ERR_* code into a Python exception carrying the library's message."""
    if rc == MI_OK:
        return
    msg = last_error()
    if rc == MI_ERR_UNSUPPORTED_SHAPE:
        raise unsupported_exc(msg)
    if rc == MI_ERR_BAD_ARG:
        raise ValueError(msg)
    raise RuntimeError(f"libmi_ns error {rc}: {msg}")
