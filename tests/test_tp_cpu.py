"""Tensor-parallel Newton-Schulz host logic on two CPU ranks (gloo): both modes and both partition dimensions must
reproduce the unsharded result on every rank.  Mirrors what the reference checks in
tests/test_distributed_muon_utils_cpu.py; nothing here touches a GPU (this build runs its kernels on one GPU only,
the sharded path is the torch operators plus all-reduce / all-gather)."""

import os
import socket
import sys

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp


def _free_port() -> int:
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _worker(rank: int, world: int, port: int, pkg_dir: str, out_dir: str) -> None:
    sys.path.insert(0, pkg_dir)
    os.environ.update(MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    torch.set_num_threads(2)
    dist.init_process_group("gloo", rank=rank, world_size=world)
    try:
        from emerging_optimizers.orthogonalized_optimizers import muon_utils

        group = dist.group.WORLD
        failures = []
        for shape in ((48, 96), (96, 48), (64, 64)):
            full = torch.randn(shape, generator=torch.Generator().manual_seed(5))
            for kind, steps in (("quintic", 5), ("cubic5", 5), ("polar_express", 6)):
                want = muon_utils.newton_schulz(full, steps=steps, coefficient_type=kind)
                for dim in (0, 1):
                    shard = full.chunk(world, dim=dim)[rank].contiguous()
                    for mode in ("duplicated", "distributed"):
                        got = muon_utils.newton_schulz_tp(shard, steps=steps, coefficient_type=kind, tp_group=group,
                                                          partition_dim=dim, tp_mode=mode)
                        err = float((got - want.chunk(world, dim=dim)[rank]).abs().max())
                        if got.shape != shard.shape or not err <= 2e-5:
                            failures.append((shape, kind, dim, mode, tuple(got.shape), err))
            # the sharded norm equals the norm of the whole
            part = muon_utils.distributed_normalize_p2(full.chunk(world, dim=0)[rank], 1e-7, group)
            if float((part - (full / full.norm()).chunk(world, dim=0)[rank]).abs().max()) > 1e-6:
                failures.append((shape, "distributed_normalize_p2"))
        with open(os.path.join(out_dir, f"rank{rank}.txt"), "w") as f:
            f.write(repr(failures))
    finally:
        dist.destroy_process_group()


@pytest.mark.timeout(180)
def test_newton_schulz_tp_matches_unsharded_on_two_ranks(tmp_path):
    pkg_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "emerging-optimizers_amd")
    mp.spawn(_worker, args=(2, _free_port(), pkg_dir, str(tmp_path)), nprocs=2, join=True)
    for rank in range(2):
        assert (tmp_path / f"rank{rank}.txt").read_text() == "[]"
