"""Python entry points of the gfx950 kernels (SYRK, GEMM+AXPY, Frobenius normalise, fused Newton-Schulz)."""

from .. import _hip
from .batched_syrk import batched_tsyrk_ex, can_use_batched_tsyrk
from .newton_schulz import (
    frob_normalize,
    fused_muon_update,
    fused_newton_schulz,
    fused_supported,
    gemm_axpy,
    on_kernel_device,
    require_library,
)
from .syrk import tsyrk_ex, tsyrk_ex_small_matrix


#: True when libmi_ns.so is loadable.  The reference's call sites test ``HAS_TRITON_340`` before taking
#: the SYRK path (muon.py:106, muon_utils.py:431,465); the same attribute name is kept for them.
HAS_HIP_KERNELS = _hip.available()
HAS_TRITON_340 = HAS_HIP_KERNELS

__all__ = [
    "HAS_HIP_KERNELS",
    "HAS_TRITON_340",
    "batched_tsyrk_ex",
    "can_use_batched_tsyrk",
    "frob_normalize",
    "fused_muon_update",
    "fused_newton_schulz",
    "fused_supported",
    "gemm_axpy",
    "on_kernel_device",
    "require_library",
    "tsyrk_ex",
    "tsyrk_ex_small_matrix",
]
