#!/usr/bin/env python3
"""Headline benchmark: Newton-Schulz orthogonalisation of one 4096 x 14336 matrix, 5 steps, bf16 kernels.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" = one full orthogonalisation (normalise, bf16 cast, 5 x {SYRK, SYRK, GEMM+AXPY}, float32 result)
of a Llama-3-8B MLP-shaped float32 gradient that is already resident in HBM.  Prints ONE JSON line:
  value       TFLOP/s on the symmetric-halved FLOP count 5 (3 m^2 n + m^3)
  roofline    the dominant kernel (GEMM+AXPY, 2 m^2 n FLOP, issued as two launches) against the bf16 dense MFMA
              peak, its duration taken from HIP events the driver records on the launch stream
  cpu_baseline the same operator sequence in float32 torch on the host cores (a baseline, not a target)
This run uses one GPU; --gpus above 1 is refused.
"""

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "emerging-optimizers_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2516.6  # MI355X dense bf16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
# HBM-side bytes of one GEMM+AXPY at the headline shape (both launches), from two `rocprofv3 --pmc` runs of this file
# (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for sumsq_kernel
# of the same run, whose traffic is known (229 376 KiB read, 114 696 KiB written): factors 1.9994 and 0.9998.
GEMM_AXPY_TRAFFIC_BYTES = int(((405915.0 + 146831.8) * 1.9994 + (98328.0 + 16392.0) * 0.9998) * 1024)
# The same for the lower-triangle kernel, averaged over its 16 launches per call (2 x X X^T, 14 m x m products).
TRI_KERNEL_TRAFFIC_BYTES = int((128715.5 * 1.9994 + 32768.1 * 0.9998) * 1024)
M, N, NS_STEPS = 4096, 14336, 5
# Other benchmark configurations, timed with --workload (the default, "mlp", is the headline).
WORKLOADS = {
    "mlp": (4096, 14336),          # Llama-3-8B MLP gradient (headline)
    "attn": (4096, 4096),          # Llama-3-8B attention projection
    "attn_x8": (8, 4096, 4096),    # eight attention projections in one batched call (multi-tensor grouping)
    "mlp_tall": (14336, 4096),     # same MLP weight stored (out, in): exercises the K-strided kernels
    "per_head": (32, 128, 4096),   # 32 heads in one grouped launch
    "moe_shard": (8, 1792, 4096),  # 8 experts, single-GPU shard shape
    "moe": (8, 4096, 14336),       # 8 stacked experts at full shape (1.9 GB of float32 gradients)
    "batched_syrk": (16, 2048, 8192),  # batched SYRK alone (no Newton-Schulz), bf16 in / bf16 out
    "muon_step": (4096, 14336),    # whole Muon.step() (momentum 0.95, Nesterov, weight decay) on the headline gradient
    "muon_heads": (32, 128, 4096),  # Muon.step() over 32 separate 128x4096 parameters: serial loop vs one batched call
}
COEFFS = [(3.4445, -4.7750, 2.0315)] * NS_STEPS  # "simple" table cycled


def llama_grad(shape, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * 1e-3
    mask = torch.rand(shape, generator=g) < 0.01
    sign = torch.where(torch.rand(shape, generator=g) < 0.5, -1.0, 1.0)
    return torch.where(mask, sign * 50e-3, x)


def cpu_baseline(x_cpu):
    """Times the torch-CPU restatement of the reference's operator sequence on a bounded sample."""
    import torch

    from oracle import ns_torch_cpu

    prev = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("highest")
    try:
        small = torch.randn(1024, 1024, generator=torch.Generator().manual_seed(0))
        for _ in range(3):
            ns_torch_cpu.newton_schulz_cpu(small, COEFFS)
        ts = []
        for _ in range(10):
            t0 = time.perf_counter()
            ns_torch_cpu.newton_schulz_cpu(small, COEFFS)
            ts.append(time.perf_counter() - t0)
        cfg1_ms = statistics.median(ts) * 1e3
        # the headline shape: one warm-up, then as many passes as fit in ~20 s (at least 1)
        t0 = time.perf_counter()
        ns_torch_cpu.newton_schulz_cpu(x_cpu, COEFFS)
        first = time.perf_counter() - t0
        reps = max(1, min(5, int(20.0 / max(first, 1e-3)) - 1))
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            ns_torch_cpu.newton_schulz_cpu(x_cpu, COEFFS)
            ts.append(time.perf_counter() - t0)
        sec = statistics.median(ts)
    finally:
        torch.set_float32_matmul_precision(prev)
    f_sym = NS_STEPS * (3 * M * M * N + M**3)
    return {
        "value": round(f_sym / sec / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{reps} timed pass(es) + 1 warm-up of the full {M}x{N} fp32 workload (torch CPU, 'highest')",
        "ms_per_step": round(sec * 1e3, 1),
        "config1_1024x1024_fp32_ms": round(cfg1_ms, 2),
        "host_cpu_count": os.cpu_count(),
    }


def batched_syrk_workload(args):
    """Batched SYRK configuration: batched_tsyrk_ex alone on 16 x (2048 x 8192) bf16, TFLOP/s on B n^2 k."""
    import torch

    from emerging_optimizers import _hip
    from emerging_optimizers.triton_kernels import batched_tsyrk_ex

    _hip.lib()
    dev = torch.device("cuda:0")
    b, n, k = WORKLOADS["batched_syrk"]
    a = (torch.randn(b, n, k, generator=torch.Generator().manual_seed(0)) * 0.02).to(torch.bfloat16).to(dev)
    out = torch.empty(b, n, n, dtype=torch.bfloat16, device=dev)
    for _ in range(args.warmup):
        batched_tsyrk_ex(a, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        batched_tsyrk_ex(a, out=out)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    ref = torch.bmm(a[:2].float(), a[:2].float().mT)
    rel = float((out[:2].float() - ref).norm() / ref.norm())
    sym = bool(torch.equal(out, out.mT))
    tflops = b * n * n * k / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "batched SYRK ms + TFLOP/s (% bf16 MFMA peak)", "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"batched_tsyrk_ex on {b}x{n}x{k} bf16 (alpha=1, beta=0), FLOPs counted B n^2 k",
                   "pct_of_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2), "rel_fro_vs_fp32": round(rel, 6),
                   "bitwise_symmetric": sym},
    }))


def muon_step_workload(args):
    """Whole optimizer step around the headline orthogonalisation: Muon(momentum 0.95, Nesterov) on one 4096 x 14336 weight."""
    import torch

    from emerging_optimizers import _hip
    from emerging_optimizers.orthogonalized_optimizers.muon import Muon

    _hip.lib()
    dev = torch.device("cuda:0")
    shape = WORKLOADS["muon_step"]
    w = torch.nn.Parameter((torch.randn(*shape, generator=torch.Generator().manual_seed(1)) * 0.02).to(dev))
    opt = Muon([w], lr=3e-4, momentum=0.95, nesterov=True, weight_decay=0.01, num_ns_steps=NS_STEPS,
               coefficient_type="simple", use_syrk=True, fp32_matmul_prec="medium")
    grads = [llama_grad(shape, seed=s).to(dev) for s in range(3)]
    for i in range(args.warmup):
        w.grad = grads[i % 3]
        opt.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        w.grad = grads[i % 3]
        opt.step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    m, n = shape
    tflops = NS_STEPS * (3 * m * m * n + m**3) / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "Muon.step ms (momentum + Nesterov + weight decay + NS orthogonalize + update)", "value": round(ms, 4),
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"Muon.step on one {m}x{n} float32 weight, llama-like gradients, lr 3e-4, momentum 0.95, "
                               "Nesterov, decoupled weight decay 0.01, 5 'simple' NS steps",
                   "ns_tflops_if_all_time_were_ns": round(tflops, 1), "finite": bool(torch.isfinite(w).all())},
    }))


def muon_heads_workload(args):
    """Muon.step over many small parameters of one shape: the reference's serial loop against group_same_shape."""
    import torch

    from emerging_optimizers import _hip
    from emerging_optimizers.orthogonalized_optimizers.muon import Muon

    _hip.lib()
    dev = torch.device("cuda:0")
    heads, m, n = WORKLOADS["muon_heads"]
    gen = torch.Generator().manual_seed(2)
    grads = [(torch.randn(heads, m, n, generator=gen) * 1e-3).to(dev) for _ in range(2)]
    ms = {}
    for grouped in (False, True):
        ps = [torch.nn.Parameter((torch.randn(m, n, generator=gen) * 0.02).to(dev)) for _ in range(heads)]
        opt = Muon(ps, lr=3e-4, momentum=0.95, nesterov=True, weight_decay=0.01, num_ns_steps=NS_STEPS,
                   coefficient_type="simple", use_syrk=True, fp32_matmul_prec="medium", group_same_shape=grouped)

        def one(i):
            for h, p in enumerate(ps):
                p.grad = grads[i % 2][h]
            opt.step()

        for i in range(args.warmup):
            one(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            one(i)
        torch.cuda.synchronize()
        ms[grouped] = (time.perf_counter() - t0) / args.steps * 1e3
    print(json.dumps({
        "metric": "Muon.step ms over 32 parameters of 128x4096 (one batched orthogonalisation per shape)",
        "value": round(ms[True], 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms[True], 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"Muon.step on {heads} separate {m}x{n} float32 weights, momentum 0.95, Nesterov, decoupled "
                               "weight decay, 5 'simple' NS steps; group_same_shape=True",
                   "ms_serial_loop": round(ms[False], 4), "speedup": round(ms[False] / ms[True], 2)},
    }))


def side_workload(args):
    """Times another benchmark configuration through the same entry point; one JSON line, no roofline legs."""
    import torch

    if args.workload == "muon_heads":
        return muon_heads_workload(args)

    if args.workload == "batched_syrk":
        return batched_syrk_workload(args)
    if args.workload == "muon_step":
        return muon_step_workload(args)

    from emerging_optimizers import _hip, utils
    from emerging_optimizers.orthogonalized_optimizers import muon_utils

    _hip.lib()
    dev = torch.device("cuda:0")
    shape = WORKLOADS[args.workload]
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(*shape, generator=gen)
    if args.workload in ("moe", "moe_shard"):  # per-expert scales log-uniform in [1e-4, 1e-2]
        lo, hi = torch.log(torch.tensor(1e-4)), torch.log(torch.tensor(1e-2))
        x = x * torch.exp(lo + (hi - lo) * torch.rand(shape[0], 1, 1, generator=gen))
    else:
        x = x * 1e-3
    x = x.to(dev)
    run = lambda: muon_utils.newton_schulz(x, steps=NS_STEPS, coefficient_type="simple", use_syrk=True)
    with utils.fp32_matmul_precision("medium"), torch.no_grad():
        for _ in range(args.warmup):
            out = run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = run()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
    torch.set_float32_matmul_precision("highest")
    nref = min(2, x.shape[0]) if x.dim() == 3 and x.numel() > (1 << 28) else None  # parity on two experts of the big batch
    if nref is not None:
        x, out = x[:nref], out[:nref]
    X = x.mT if x.shape[-2] > x.shape[-1] else x
    X = X / X.norm(dim=(-2, -1), keepdim=True)
    for a, b, c in COEFFS:
        A = X @ X.mT
        X = a * X + (b * A + c * (A @ A)) @ X
    ref = X.mT if x.shape[-2] > x.shape[-1] else X
    rel = float((out.double() - ref.double()).norm() / ref.double().norm())
    batch = shape[0] if len(shape) == 3 else 1
    m, n = sorted(shape[-2:])
    f_sym = batch * NS_STEPS * (3 * m * m * n + m**3)
    tflops = f_sym / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "NS orthogonalize ms + TFLOP/s (% bf16 MFMA peak)", "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"newton_schulz {NS_STEPS} steps on {'x'.join(map(str, shape))} ({args.workload})",
                   "pct_of_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2), "rel_fro_vs_fp32": round(rel, 6)},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-core baseline leg")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="mlp", help="benchmark configuration to time")
    args = ap.parse_args()
    if args.workload != "mlp":
        return side_workload(args)
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus above 1 is not supported (no collectives are built).")

    import torch

    from emerging_optimizers import _hip, hip_kernels, utils
    from emerging_optimizers.orthogonalized_optimizers import muon_utils

    lib = _hip.lib()  # fails loudly if the kernels are missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    x_cpu = llama_grad((M, N), seed=0)
    x = x_cpu.to(dev)

    def run():
        return muon_utils.newton_schulz(x, steps=NS_STEPS, coefficient_type="simple", use_syrk=True)

    with utils.fp32_matmul_precision("medium"), torch.no_grad():
        for _ in range(args.warmup):
            out = run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = run()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

        # per-kernel durations over another K steps, from HIP events recorded on the launch stream
        lib.mi_profile_begin()
        for _ in range(args.steps):
            out = run()
        ms_kind = (ctypes.c_float * 4)()
        n_kind = (ctypes.c_int * 4)()
        _hip.check(lib.mi_profile_end(ms_kind, n_kind))

    ms_per_step = elapsed / args.steps * 1e3
    f_sym = NS_STEPS * (3 * M * M * N + M**3)
    f_full = NS_STEPS * (4 * M * M * N + 2 * M**3)
    tflops = f_sym / (ms_per_step * 1e-3) / 1e12
    # What the driver executes: wide matrices take the five steps as 3 + 2 (2 + 1 + 2 under MI_NS_PAIRS=pairs), where a
    # group of g steps shares one X X^T and one B X and pays 4 g - 3 symmetric m x m products (same result within the
    # tolerance, checked below against float32).  MI_NS_PAIRS=0 restores one X X^T and one B X per step.
    env = os.environ.get("MI_NS_PAIRS", "")[:1]
    wide = M >= 1024 and N >= 2 * M and NS_STEPS == 5
    schedule = [1] * NS_STEPS if (env == "0" or not wide) else [2, 1, 2] if env in ("p", "f") else [3, 2]
    f_exec = sum(3 * M * M * N + (4 * g - 3) * M**3 for g in schedule)
    # parity gate in the same job: float32 Newton-Schulz with torch on the GPU
    torch.set_float32_matmul_precision("highest")
    X = x / x.norm()
    for a, b, c in COEFFS:
        A = X @ X.mT
        X = a * X + (b * A + c * (A @ A)) @ X
    rel = float((out.double() - X.double()).norm() / X.double().norm())
    del X, A

    names = ["normalize_cast", "syrk_gram", "syrk_poly", "gemm_axpy"]
    per_kernel = {n: (ms_kind[i] / n_kind[i] if n_kind[i] else None) for i, n in enumerate(names)}
    gemm_ms = per_kernel["gemm_axpy"]
    gemm_flop = 2.0 * M * M * N  # algorithmic FLOP of one GEMM+AXPY launch pair
    gemm_tflops = gemm_flop / (gemm_ms * 1e-3) / 1e12 if gemm_ms else None
    # The kernel with the largest share of the GPU time is the lower-triangle kernel (one rocprof row: 192 x 192
    # tiles), which serves X X^T (m^2 n FLOP sym-halved) and every m x m product (m^3 FLOP): its launches are
    # priced together, algorithmic FLOP per launch over the average launch duration.
    tri_launches = n_kind[1] + n_kind[2]
    tri_ms = (ms_kind[1] + ms_kind[2]) / tri_launches if tri_launches else None
    tri_flop = (n_kind[1] * float(M) * M * N + n_kind[2] * float(M) ** 3) / tri_launches if tri_launches else None
    achieved = tri_flop / (tri_ms * 1e-3) / 1e12 if tri_ms else None
    line = {
        "metric": "NS orthogonalize ms + TFLOP/s (% bf16 MFMA peak) at 4096x14336 bf16",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"newton_schulz, {NS_STEPS} steps ('simple' coefficients), one {M}x{N} float32 gradient "
            "(N(0,1e-3^2) with 1% entries at 50 sigma), bf16 MFMA kernels with fp32 accumulation, float32 result",
            "flops_counted": "symmetric-halved 5*(3 m^2 n + m^3): the count of five ordinary steps, whatever the schedule",
            "tflops_full_count": round(f_full / (ms_per_step * 1e-3) / 1e12, 2),
            "schedule": "+".join(map(str, schedule)) + " (steps of one group share one Gram matrix)",
            "tflops_executed": round(f_exec / (ms_per_step * 1e-3) / 1e12, 2),
            "pct_of_bf16_mfma_peak_executed": round(100.0 * f_exec / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 2),
            "launches_per_call": {n: n_kind[i] // args.steps for i, n in enumerate(["normalize_cast", "syrk_gram", "syrk_poly", "gemm_axpy"])},
            "pct_of_bf16_mfma_peak": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
            "rel_fro_vs_fp32": round(rel, 6),
            "tolerance": 1e-2,
            "kernel_ms": {k: (round(v, 4) if v is not None else None) for k, v in per_kernel.items()},
            "gemm_axpy_tflops": round(gemm_tflops, 1) if gemm_tflops else None,
            "gemm_axpy_traffic_bytes": GEMM_AXPY_TRAFFIC_BYTES if (M, N) == (4096, 14336) else None,
        },
        "roofline": {
            "kernel": "gemm_fast_kernel<FastCfg<192,...>, SYRK mode> (lower-triangle kernel: X X^T and the m x m products; "
            f"{n_kind[1] // args.steps} + {n_kind[2] // args.steps} launches per call, sym-halved FLOP, average launch)",
            "bound": "mfma",
            "achieved": round(achieved, 2) if achieved else None,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4) if achieved else None,
            "traffic": TRI_KERNEL_TRAFFIC_BYTES if ((M, N) == (4096, 14336) and schedule == [3, 2]) else None,
            "avg_launch_ms": round(tri_ms, 4) if tri_ms else None,
        },
    }
    if rel > 1e-2:
        line["config"]["parity"] = "FAILED"
    line["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline(x_cpu)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
