"""Shared launch plumbing: tensors -> raw pointers/strides -> C ABI call on the current stream."""

from __future__ import annotations

import ctypes

import torch

from .. import _hip


def ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def require_gpu(t: torch.Tensor, who: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{who} runs on the GPU only; got a tensor on {t.device}")


# One cached scratch buffer per (device, stream): calls on one stream are serialised by the stream itself, so they can
# share scratch; different streams get different buffers.
_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, device=device, dtype=torch.uint8)
        _workspaces[key] = ws
    return ws


def syrk_launch(
    mem_a: torch.Tensor,
    a_trans: bool,
    batch: int,
    n: int,
    k: int,
    c_mem: torch.Tensor | None,
    alpha: float,
    beta: float,
    d: torch.Tensor,
    skip_upper: bool,
) -> None:
    """``mem_a`` is the contiguous view of the operand: (B?, n, k) when not a_trans, else (B?, k, n)."""
    lib = _hip.lib()
    with torch.cuda.device(d.device):
        # scratch for the stream-K launch, when the library would use one for this shape
        nbytes = 0 if skip_upper else lib.mi_syrk_workspace_bytes(batch, n, k, int(a_trans))
        ws = workspace(d.device, nbytes) if nbytes else None
        rc = lib.mi_syrk_bf16_ws(
            ptr(mem_a), batch, n, k, n * k, mem_a.shape[-1], int(a_trans),
            ptr(c_mem), n * n, n, float(alpha), float(beta),
            ptr(d), n * n, n, int(bool(skip_upper)), ptr(ws), ws.numel() if ws is not None else 0,
            _hip.current_stream_ptr(d.device),
        )  # fmt: skip
    _hip.check(rc)
