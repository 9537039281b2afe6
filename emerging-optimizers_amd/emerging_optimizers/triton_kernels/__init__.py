"""Import-path alias: the reference keeps its SYRK kernels in ``emerging_optimizers.triton_kernels``.

Nothing here uses Triton.  The names resolve to the HIP implementations in ``hip_kernels`` so that
``triton_kernels.tsyrk_ex`` / ``batched_tsyrk_ex`` / ``HAS_TRITON_340`` call sites need no edit.
"""

from ..hip_kernels import (  # noqa: F401
    HAS_HIP_KERNELS,
    HAS_TRITON_340,
    batched_tsyrk_ex,
    can_use_batched_tsyrk,
    tsyrk_ex,
    tsyrk_ex_small_matrix,
)

__all__ = ["HAS_TRITON_340", "batched_tsyrk_ex", "can_use_batched_tsyrk", "tsyrk_ex", "tsyrk_ex_small_matrix"]
