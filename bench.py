#!/usr/bin/env python3
"""Benchmark of the Muon orthogonalisation path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline] [--no-others] [--data zeros] [--torch-comparators]

Headline (the default): Newton-Schulz orthogonalisation of one 4096 x 14336 float32 gradient that is already resident
in HBM: normalise, bf16 cast, 5 quintic steps on the bf16 MFMA kernels, float32 result.  One "step" of the benchmark is
one such orthogonalisation.  The run prints ONE JSON line:
  value        TFLOP/s on the symmetric-halved FLOP count of five ordinary steps, 5 (3 m^2 n + m^3); ms_per_step is the
               wall clock of exactly K steps between two device synchronisations, divided by K
  config       median and minimum over per-step HIP event pairs, the schedule the driver executed and its FLOPs, the
               float32 parity gate, per-kernel times, and `other_workloads`: every other benchmark configuration
               (attention shape, batched SYRK alone and the reference's own SYRK benchmark shapes, per-head batch,
               expert stacks, whole Muon.step) timed in the same process with >= 3 warm-up and >= 20 timed iterations
  roofline     the kernel with the largest share of the GPU time (the lower-triangle product kernel, which serves
               X X^T and every m x m product): algorithmic (symmetric-halved) FLOP per launch over its average launch
               duration, taken from HIP events the library records on the launch stream; `frac_executed` prices the
               MFMA work the launches really issue (whole tiles, idle quarter of diagonal tiles left out)
  cpu_baseline the same operator sequence in float32 torch on the host cores (a baseline, not a target); timed first,
               so that the GPU work ends the run
Stated baselines beside the kernels (never targets), timed in the same process with the same warm-up and iteration
counts, only with --torch-comparators: the Newton-Schulz rows `mlp` and `attn` carry `torch_bf16_path_ms`, the reference's own operator sequence with
use_syrk=False (normalise, bf16 cast, X @ X.mT / addmm / addmm per step, float32 cast) on torch's GPU operators --
what the reference executes on this GPU, whose SYRK gate admits NVIDIA parts only; the `batched_syrk` row carries
`torch_bmm_ms` and `torch_baddbmm_ms` (for its beta variant), and every SYRK row `beta_variant_ms` and
`loop_single_ms`, a Python loop of single-matrix calls, as the reference's SYRK benchmark times them
(benchmarks/bench_batched_syrk.py:71-96 there).  Without the flag, and on the other rows, the torch figures are
null: see TORCH_COMPARATOR_ROWS for why torch's bf16 matmuls are not part of the default run.
A parity gate that fails (relative Frobenius error against float32 above 1e-2, or a SYRK result that is not bitwise
symmetric) is reported in the line and makes the process exit with status 1.  This build runs on one GPU; --gpus
above 1 is refused.
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
PEAK_HBM_GBPS = 8000.0
TOL = 1e-2
# HBM-side bytes per launch of the lower-triangle kernel at the headline shape, averaged over its 16 launches per call
# (2 x X X^T, 14 m x m products), and of one GEMM+AXPY (both launches): FETCH_SIZE and WRITE_SIZE of two
# `rocprofv3 --pmc` runs of this file (KiB per dispatch), each scaled by what the same counter reads for sumsq_kernel
# of the same run, whose traffic is known (229 376 KiB read, 114 696 KiB written): factors 1.9994 and 0.9998.
TRAFFIC_SOURCE = ("profiles/newton_schulz_4096x14336_pmc.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command; a constant "
                  "from that profile, not measured in this run; null when tile choice or schedule differ from the profiled ones)")
TRI_KERNEL_TRAFFIC_BYTES = int((129117.8 * 1.9994 + 32768.0 * 0.9998) * 1024)
GEMM_AXPY_TRAFFIC_BYTES = int(((407572.7 + 146821.6) * 1.9994 + (98328.0 + 16392.0) * 0.9998) * 1024)
M, N, NS_STEPS = 4096, 14336, 5
COEFFS = [(3.4445, -4.7750, 2.0315)] * NS_STEPS  # "simple" table cycled
MIN_WARMUP, MIN_TIMED = 3, 20
# Comparators on torch's own bf16 matmuls (hipBLASLt through torch 2.10 / ROCm 7.2 of this image) are timed only with
# --torch-comparators, and then only on these rows.  Of six benchmark runs that called torch's bf16 matmuls, three ended
# with a GPU memory fault that took the whole box down: one inside ns_torch_bf16_path on the 8 x 1792 x 4096 stack,
# with none of this library's kernels in flight, two at a place that could not be read back; no run without them
# faulted, on the same kernels, before or after.  The default run therefore calls no torch bf16 matmul at all (its
# float32 parity references are torch float32 matmuls, as in every earlier run).  The figures of the one complete run
# with comparators are kept under profiles/ (bench_all_workloads_with_torch_comparators).
TORCH_COMPARATOR_ROWS = ("mlp", "attn", "batched_syrk")
TORCH_COMPARATORS = False  # set by --torch-comparators

# name -> shape.  "mlp" is the headline; the others are timed after it (or alone with --workload).
NS_WORKLOADS = {
    "mlp": (4096, 14336),          # Llama-3-8B MLP gradient (headline)
    "attn": (4096, 4096),          # Llama-3-8B attention projection
    "mlp_tall": (14336, 4096),     # the same MLP weight stored (out, in): transposed inside the bf16 cast
    "per_head": (32, 128, 4096),   # 32 heads in one grouped launch
    "moe_shard": (8, 1792, 4096),  # 8 experts, single-GPU shard shape
    "moe": (8, 4096, 14336),       # 8 stacked experts at full shape (1.9 GB of float32 gradients)
    "attn_x8": (8, 4096, 4096),    # eight attention projections in one batched call
}
# batched SYRK alone: the benchmark configuration first, then the other shapes of the reference's own SYRK benchmark
# (benchmarks/bench_batched_syrk.py:104-110 there)
SYRK_WORKLOADS = {
    "batched_syrk": (16, 2048, 8192),
    "syrk_8x2048x2048": (8, 2048, 2048),
    "syrk_4x4096x4096": (4, 4096, 4096),
    "syrk_32x512x2048": (32, 512, 2048),
    "syrk_64x256x1024": (64, 256, 1024),
    # the Gram product of the headline shape alone, operand stored row-major (K-contiguous) and transposed (K-strided:
    # the reference's TRANS layout, triton_kernels/syrk.py:200-207 there)
    "syrk_4096x14336": (1, 4096, 14336),
    "syrk_4096x14336_trans": (1, 4096, 14336),
}
STEP_WORKLOADS = {
    "muon_step": (4096, 14336),      # whole Muon.step() (momentum 0.95, Nesterov, weight decay) on the headline gradient
    "muon_step_attn": (4096, 4096),
    "muon_heads": (32, 128, 4096),   # Muon.step() over 32 separate 128 x 4096 parameters, one batched orthogonalisation
    "muon_step_default": (4096, 14336),  # Muon(params) with every argument at the reference's default (use_syrk=False, "quintic")
}
DEFAULT_OTHERS = ["attn", "batched_syrk", "per_head", "moe_shard", "moe", "muon_step", "muon_step_default", "muon_step_attn", "mlp_tall",
                  "syrk_8x2048x2048", "syrk_4x4096x4096", "syrk_32x512x2048", "syrk_64x256x1024", "syrk_4096x14336",
                  "syrk_4096x14336_trans", "muon_heads"]
ALL_WORKLOADS = list(NS_WORKLOADS) + list(SYRK_WORKLOADS) + list(STEP_WORKLOADS)


def llama_grad(shape, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * 1e-3
    mask = torch.rand(shape, generator=g) < 0.01
    sign = torch.where(torch.rand(shape, generator=g) < 0.5, -1.0, 1.0)
    return torch.where(mask, sign * 50e-3, x)


def note(msg):
    """Progress line on stderr, flushed before the GPU step it names: a run that dies on the GPU still says where."""
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def time_events(fn, warmup, iters):
    """(wall ms per iteration over exactly `iters` calls between two synchronisations, [per-iteration ms from HIP event
    pairs on the current stream]).  No host synchronisation inside the timed region."""
    import torch

    for _ in range(warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(iters):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / iters * 1e3
    return wall, [s.elapsed_time(e) for s, e in zip(starts, stops)]


def ns_fp32_reference(x):
    """float32 Newton-Schulz with torch on the GPU ("highest" matmul precision): the parity reference."""
    import torch

    prev = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("highest")
    try:
        tall = x.shape[-2] > x.shape[-1]
        X = x.mT if tall else x
        X = X / X.norm(dim=(-2, -1), keepdim=True)
        for a, b, c in COEFFS:
            A = X @ X.mT
            X = a * X + (b * A + c * (A @ A)) @ X
        return X.mT if tall else X
    finally:
        torch.set_float32_matmul_precision(prev)


def ns_torch_bf16_path(x, coeffs):
    """The reference's operator sequence under "medium" with use_syrk=False (muon_utils.py:212-273, 370-377, 403-410
    there) on torch's own GPU operators: a stated baseline, what the reference would execute on this GPU."""
    import torch

    tall = x.shape[-2] > x.shape[-1]
    X = x.mT if tall else x
    X = torch.nn.functional.normalize(X, p=2, dim=(-2, -1), eps=1e-15).to(torch.bfloat16)
    add = torch.baddbmm if X.dim() == 3 else torch.addmm
    for a, b, c in coeffs:
        A = X @ X.mT
        X = add(X, add(A, A, A, alpha=c, beta=b), X, alpha=1.0, beta=a)
    X = X.to(torch.float32)
    return X.mT if tall else X


def schedule_of(lib, batch, rows, cols):
    abc = (ctypes.c_float * (3 * NS_STEPS))(*[v for c in COEFFS for v in c])
    out = (ctypes.c_int * 16)()
    count = lib.mi_newton_schulz_schedule(batch, rows, cols, abc, NS_STEPS, out, 16)
    return list(out[:count])


def ns_flops(batch, m, n, schedule):
    """(symmetric-halved FLOPs of five ordinary steps, full count, symmetric-halved FLOPs of the executed schedule: a
    group of g steps costs one X X^T, one B X and 4 g - 3 products of symmetric m x m matrices)."""
    f_sym = batch * NS_STEPS * (3 * m * m * n + m**3)
    f_full = batch * NS_STEPS * (4 * m * m * n + 2 * m**3)
    f_exec = batch * sum(3 * m * m * n + (4 * g - 3) * m**3 for g in schedule)
    return f_sym, f_full, f_exec


def ns_input(name, shape, dev):
    import torch

    if name in ("mlp", "attn", "mlp_tall"):
        return llama_grad(shape, seed=0).to(dev)
    gen = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(*shape, device=dev, generator=gen)
    if name in ("moe", "moe_shard"):  # per-expert scales log-uniform in [1e-4, 1e-2]
        cg = torch.Generator().manual_seed(0)
        lo, hi = torch.log(torch.tensor(1e-4)), torch.log(torch.tensor(1e-2))
        return x * torch.exp(lo + (hi - lo) * torch.rand(shape[0], 1, 1, generator=cg)).to(dev)
    return x * 1e-3


def run_ns_workload(name, warmup, iters, lib, dev, zeros=False):
    """newton_schulz on one benchmark shape: timing, executed schedule, parity against float32."""
    import torch

    from emerging_optimizers import utils
    from emerging_optimizers.orthogonalized_optimizers import muon_utils

    shape = NS_WORKLOADS[name]
    note(f"{name}: newton_schulz on {shape}, kernels")
    x = torch.zeros(*shape, device=dev) if zeros else ns_input(name, shape, dev)
    run = lambda: muon_utils.newton_schulz(x, steps=NS_STEPS, coefficient_type="simple", use_syrk=True)
    with utils.fp32_matmul_precision("medium"), torch.no_grad():
        wall, per = time_events(run, warmup, iters)
        out = run()
    batch = shape[0] if len(shape) == 3 else 1
    m, n = sorted(shape[-2:])
    schedule = schedule_of(lib, batch, shape[-2], shape[-1])
    f_sym, f_full, f_exec = ns_flops(batch, m, n, schedule)
    # stated baseline: the reference's own bf16 operator sequence on torch's operators, same counts
    torch_ms = torch_rel = None
    compare = TORCH_COMPARATORS and not zeros and name in TORCH_COMPARATOR_ROWS
    if compare:
        note(f"{name}: the reference's bf16 operator sequence on torch's operators")
        with torch.no_grad():
            _, tper = time_events(lambda: ns_torch_bf16_path(x, COEFFS), warmup, iters)
            tout = ns_torch_bf16_path(x, COEFFS)
        torch_ms = statistics.median(tper)
    note(f"{name}: parity against float32")
    # parity: every matrix of a batch (two of them for the 1.9 GB stack)
    idx = range(batch) if x.dim() == 3 and x.numel() <= (1 << 28) else (range(2) if x.dim() == 3 else [None])
    rels = [0.0] if zeros else []
    trels = []
    for i in ([] if zeros else idx):
        xi, oi = (x, out) if i is None else (x[i], out[i])
        ref = ns_fp32_reference(xi)
        rels.append(float((oi.double() - ref.double()).norm() / ref.double().norm()))
        if compare:
            ti = tout if i is None else tout[i]
            trels.append(float((ti.double() - ref.double()).norm() / ref.double().norm()))
        del ref
    if compare:
        torch_rel = max(trels)
        del tout
    med, mn = statistics.median(per), min(per)
    res = {
        "workload": f"newton_schulz {NS_STEPS} steps on {'x'.join(map(str, shape))} float32 ({name})",
        "ms_median": round(med, 4), "ms_min": round(mn, 4), "ms_wall": round(wall, 4), "iters": iters,
        "tflops_sym": round(f_sym / med / 1e9, 1),
        "pct_peak": round(100 * f_sym / med / 1e9 / PEAK_BF16_TFLOPS, 2),
        "schedule": "+".join(map(str, schedule)),
        "pct_peak_executed": round(100 * f_exec / med / 1e9 / PEAK_BF16_TFLOPS, 2),
        "rel_fro": round(max(rels), 6), "parity": "ok" if max(rels) <= TOL else "FAILED",
        "torch_bf16_path_ms": round(torch_ms, 4) if torch_ms else None,
        "speedup_vs_torch": round(torch_ms / med, 2) if torch_ms else None,
        "torch_bf16_path_rel_fro": round(torch_rel, 6) if torch_rel is not None else None,
    }
    if name == "per_head":
        # memory-bound: algorithmic bytes = float32 in and out once, and per step two reads and one write of the bf16 copy
        algo = batch * m * n * (4 + 4 + NS_STEPS * 3 * 2)
        res["gbps"] = round(algo / med / 1e6, 1)
        res["pct_hbm_peak"] = round(100 * algo / med / 1e6 / PEAK_HBM_GBPS, 2)
        res["algorithmic_bytes"] = algo
    return res, (wall, per, out, x, schedule)


def run_syrk_workload(name, warmup, iters, dev):
    """batched_tsyrk_ex alone: bf16 in, bf16 out, alpha = 1, beta = 0; FLOPs counted B n^2 k (symmetric-halved)."""
    import torch

    from emerging_optimizers.triton_kernels import batched_tsyrk_ex

    b, n, k = SYRK_WORKLOADS[name]
    note(f"{name}: batched_tsyrk_ex on {b}x{n}x{k}")
    a = (torch.randn(b, n, k, device=dev, generator=torch.Generator(device=dev).manual_seed(0)) * 0.02).to(torch.bfloat16)
    trans = name.endswith("_trans")
    if trans:
        a = a.mT.contiguous().mT  # same values, stored as k rows of n
    out = torch.empty(b, n, n, dtype=torch.bfloat16, device=dev)
    wall, per = time_events(lambda: batched_tsyrk_ex(a, out=out), warmup, iters)
    nref = min(b, 2)
    ref = torch.bmm(a[:nref].float(), a[:nref].float().mT)
    rel = float((out[:nref].float() - ref).norm() / ref.norm())
    sym = bool(torch.equal(out, out.mT))
    med, mn = statistics.median(per), min(per)
    flop = b * n * n * k
    # stated baselines, as the reference's SYRK benchmark times them (benchmarks/bench_batched_syrk.py:71-96 there):
    # torch.bmm / torch.baddbmm on the same operands, the beta variant of the kernel, a loop of single-matrix calls
    from emerging_optimizers.triton_kernels import tsyrk_ex

    cmat = out.clone()  # a symmetric bf16 addend
    bmm_ms = baddbmm_ms = None
    if TORCH_COMPARATORS and name in TORCH_COMPARATOR_ROWS:
        note(f"{name}: torch.bmm / torch.baddbmm")
        bmm_ms = statistics.median(time_events(lambda: torch.bmm(a, a.mT), warmup, iters)[1])
        baddbmm_ms = statistics.median(time_events(lambda: torch.baddbmm(cmat, a, a.mT, alpha=0.5, beta=0.25), warmup, iters)[1])
    note(f"{name}: beta variant")
    beta_ms = statistics.median(time_events(lambda: batched_tsyrk_ex(a, cmat, alpha=0.5, beta=0.25, out=out), warmup, iters)[1])
    want = torch.baddbmm(cmat[:nref].float(), a[:nref].float(), a[:nref].float().mT, alpha=0.5, beta=0.25)
    rel_beta = float((out[:nref].float() - want).norm() / want.norm())
    sym = sym and bool(torch.equal(out, out.mT))
    rel = max(rel, rel_beta)
    note(f"{name}: loop of {b} single-matrix calls")
    loop_ms = statistics.median(time_events(lambda: [tsyrk_ex(a[i]) for i in range(b)], warmup, iters)[1])
    extra = {
        "torch_bmm_ms": round(bmm_ms, 4) if bmm_ms else None, "speedup_vs_torch": round(bmm_ms / med, 2) if bmm_ms else None,
        "beta_variant_ms": round(beta_ms, 4), "torch_baddbmm_ms": round(baddbmm_ms, 4) if baddbmm_ms else None,
        "beta_speedup_vs_torch": round(baddbmm_ms / beta_ms, 2) if baddbmm_ms else None, "loop_single_ms": round(loop_ms, 4),
    }
    return {**{
        "workload": f"batched_tsyrk_ex on {b}x{n}x{k} bf16{', operand stored transposed' if trans else ''} ({name})",
        "ms_median": round(med, 4), "ms_min": round(mn, 4), "ms_wall": round(wall, 4), "iters": iters,
        "tflops_sym": round(flop / med / 1e9, 1), "pct_peak": round(100 * flop / med / 1e9 / PEAK_BF16_TFLOPS, 2),
        "rel_fro": round(rel, 6), "bitwise_symmetric": sym, "parity": "ok" if (rel <= TOL and sym) else "FAILED",
    }, **extra}


def step_update_error(opt_cls, kw, w, opt, grad):
    """One more step of `opt` on `w`, beside the same step taken statement by statement in float32 ("highest" matmul
    precision, torch operators only) from a copy of the same state: relative Frobenius distance of the two updates."""
    import torch

    q = torch.nn.Parameter(w.detach().clone())
    ref = opt_cls([q], **{**kw, "fp32_matmul_prec": "highest", "use_syrk": False})
    ref.state[q]["momentum_buffer"] = opt.state[w]["momentum_buffer"].clone()
    group = opt.param_groups[0]
    lr, wd = group["lr"], group["weight_decay"]
    before = w.detach().clone()
    w.grad, q.grad = grad, grad.clone()
    opt.step()
    ref.step()
    got = w.detach() - before * (1 - lr * wd)   # decoupled weight decay
    want = q.detach() - before * (1 - lr * wd)
    return float((got.double() - want.double()).norm() / want.double().norm())


def run_step_workload(name, warmup, iters, dev):
    """Whole Muon.step (momentum 0.95, Nesterov, decoupled weight decay 0.01, 5 'simple' steps); `muon_step_default`:
    Muon(params) with every argument at the reference's default (use_syrk=False, 'quintic', no Nesterov)."""
    import torch

    from emerging_optimizers.orthogonalized_optimizers.muon import Muon

    shape = STEP_WORKLOADS[name]
    note(f"{name}: Muon.step on {shape}")
    kw = dict(lr=3e-4, momentum=0.95, nesterov=True, weight_decay=0.01, num_ns_steps=NS_STEPS, coefficient_type="simple",
              use_syrk=True, fp32_matmul_prec="medium")
    if name == "muon_step_default":
        kw = {}
    if name == "muon_heads":
        heads, m, n = shape
        gen = torch.Generator(device=dev).manual_seed(2)
        grads = [torch.randn(heads, m, n, device=dev, generator=gen) * 1e-3 for _ in range(2)]
        res = {}
        finals = {}
        for grouped in (False, True):
            gen_w = torch.Generator(device=dev).manual_seed(3)
            ps = [torch.nn.Parameter(torch.randn(m, n, device=dev, generator=gen_w) * 0.02) for _ in range(heads)]
            opt = Muon(ps, group_same_shape=grouped, **kw)
            state = {"i": 0}

            def one():
                for h, p in enumerate(ps):
                    p.grad = grads[state["i"] % 2][h]
                state["i"] += 1
                opt.step()

            _, per = time_events(one, warmup, iters)
            res[grouped] = (statistics.median(per), min(per))
            finals[grouped] = torch.stack([p.detach() for p in ps])
        # same weights, same gradients, same number of steps: the grouped step must land where the serial loop does.
        # (Not bit for bit: the serial loop takes the one-call update per weight, whose momentum and weight arithmetic
        # runs inside the kernels, the grouped step takes torch's multi-tensor statements around one batched
        # orthogonalisation; they differ by float32 rounding of the elementwise parts, and a direction that differs in
        # its last bit moves a few bf16 roundings.  Measured 6e-5 after 23 steps.)
        drift = float((finals[True] - finals[False]).norm() / finals[False].norm())
        return {
            "workload": f"Muon.step over {heads} separate {m}x{n} float32 weights, group_same_shape=True ({name})",
            "ms_median": round(res[True][0], 4), "ms_min": round(res[True][1], 4), "iters": iters,
            "ms_median_serial_loop": round(res[False][0], 4), "rel_fro_vs_serial_loop": round(drift, 8),
            "parity": "ok" if drift <= 1e-3 and bool(torch.isfinite(finals[True]).all()) else "FAILED",
        }
    w = torch.nn.Parameter((torch.randn(*shape, generator=torch.Generator().manual_seed(1)) * 0.02).to(dev))
    opt = Muon([w], **kw)
    grads = [llama_grad(shape, seed=s).to(dev) for s in range(3)]
    state = {"i": 0}

    def one():
        w.grad = grads[state["i"] % 3]
        state["i"] += 1
        opt.step()

    wall, per = time_events(one, warmup, iters)
    med, mn = statistics.median(per), min(per)
    note(f"{name}: update against the float32 statements")
    rel = step_update_error(Muon, kw, w, opt, grads[0])
    m, n = sorted(shape)
    # elementwise traffic of the step outside the products: gradient and momentum read, momentum written, bf16 cast
    # written, weight read and written
    elementwise = m * n * (4 + 4 + 4 + 2 + 4 + 4)
    what = "all arguments at the reference's defaults (use_syrk=False, quintic)" if name == "muon_step_default" else "llama-like gradients, warmed buffer"
    return {
        "workload": f"Muon.step on one {'x'.join(map(str, shape))} float32 weight, {what} ({name})",
        "ms_median": round(med, 4), "ms_min": round(mn, 4), "ms_wall": round(wall, 4), "iters": iters,
        "elementwise_bytes": elementwise, "update_rel_fro_vs_fp32_statements": round(rel, 6),
        "parity": "ok" if (rel <= TOL and bool(torch.isfinite(w).all())) else "FAILED",
    }


def run_other(name, warmup, iters, lib, dev):
    if name in NS_WORKLOADS:
        return run_ns_workload(name, warmup, iters, lib, dev)[0]
    if name in SYRK_WORKLOADS:
        return run_syrk_workload(name, warmup, iters, dev)
    return run_step_workload(name, warmup, iters, dev)


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


def tri_kernel_executed_flop(lib, dev, n, k):
    """MFMA FLOP one lower-triangle launch on (n x k) issues: whole tiles of the size the library picks for this
    shape, minus the quarter of every diagonal tile whose wavefront sits the product out."""
    import torch

    from emerging_optimizers import _hip
    from emerging_optimizers.triton_kernels import tsyrk_ex

    a = torch.zeros(n, k, dtype=torch.bfloat16, device=dev)
    tsyrk_ex(a)
    tile = _hip.last_launch()["tile_m"]
    t = -(-n // tile)
    return (t * (t - 1) / 2 + 0.75 * t) * tile * tile * k * 2.0, tile


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-core baseline leg")
    ap.add_argument("--no-others", action="store_true", help="headline only: skip the other benchmark configurations")
    ap.add_argument("--workload", choices=ALL_WORKLOADS, default="mlp", help="time this configuration alone")
    ap.add_argument("--torch-comparators", action="store_true",
                    help="also time torch's own bf16 matmuls beside the kernels on the rows mlp, attn and batched_syrk (off by "
                         "default: see TORCH_COMPARATOR_ROWS)")
    ap.add_argument("--data", choices=["synthetic", "zeros"], default="synthetic",
                    help="zeros: all-zero headline input (a power probe: the matrix pipes then toggle no operand bits and "
                         "the clock stays up; no parity gate, no other workloads)")
    args = ap.parse_args()
    global TORCH_COMPARATORS
    TORCH_COMPARATORS = args.torch_comparators
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus above 1 is not supported (no collectives are built).")

    import torch

    from emerging_optimizers import _hip

    lib = _hip.lib()  # fails loudly if the kernels are missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload != "mlp":
        res = run_other(args.workload, max(args.warmup, MIN_WARMUP), max(args.steps, MIN_TIMED), lib, dev)
        unit_ms = "tflops_sym" not in res
        print(json.dumps({
            "metric": "ms per call" if unit_ms else "TFLOP/s (symmetric-halved FLOPs) and % of the bf16 MFMA peak",
            "value": res["ms_median"] if unit_ms else res["tflops_sym"], "unit": "ms" if unit_ms else "TFLOP/s", "n_gpus": 1,
            "steps": max(args.steps, MIN_TIMED), "warmup": max(args.warmup, MIN_WARMUP), "ms_per_step": res["ms_median"],
            "higher_is_better": not unit_ms, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": res,
        }))
        sys.exit(0 if res["parity"] == "ok" else 1)

    # ---- headline ----
    zeros = args.data == "zeros"
    if zeros:
        args.no_others = args.no_cpu_baseline = True
    # the host-core baseline goes first: the GPU work then ends the run
    note("host-core baseline (CPU only)")
    cpu_line = None if args.no_cpu_baseline else cpu_baseline(llama_grad((M, N), seed=0))
    res, (wall_ms, per, out, x, schedule) = run_ns_workload("mlp", args.warmup, args.steps, lib, dev, zeros=zeros)
    from emerging_optimizers import utils
    from emerging_optimizers.orthogonalized_optimizers import muon_utils

    # per-kernel durations over another K steps, from HIP events the library records on the launch stream
    note("mlp: per-kernel event pass")
    with utils.fp32_matmul_precision("medium"), torch.no_grad():
        lib.mi_profile_begin()
        for _ in range(args.steps):
            muon_utils.newton_schulz(x, steps=NS_STEPS, coefficient_type="simple", use_syrk=True)
        ms_kind = (ctypes.c_float * 4)()
        n_kind = (ctypes.c_int * 4)()
        _hip.check(lib.mi_profile_end(ms_kind, n_kind))
    del out
    f_sym, f_full, f_exec = ns_flops(1, M, N, schedule)
    tflops = f_sym / wall_ms / 1e9
    names = ["normalize_cast", "syrk_gram", "syrk_poly", "gemm_axpy"]
    per_kernel = {n: (ms_kind[i] / n_kind[i] if n_kind[i] else None) for i, n in enumerate(names)}
    gemm_ms = per_kernel["gemm_axpy"]
    gemm_tflops = 2.0 * M * M * N / gemm_ms / 1e9 if gemm_ms else None
    # The lower-triangle kernel serves X X^T (m^2 n FLOP symmetric-halved) and every m x m product (m^3 FLOP): its
    # launches are priced together, algorithmic FLOP per launch over the average launch duration.
    tri_launches = n_kind[1] + n_kind[2]
    tri_ms = (ms_kind[1] + ms_kind[2]) / tri_launches if tri_launches else None
    tri_flop = (n_kind[1] * float(M) * M * N + n_kind[2] * float(M) ** 3) / tri_launches if tri_launches else None
    achieved = tri_flop / tri_ms / 1e9 if tri_ms else None
    ex_gram, tile_gram = tri_kernel_executed_flop(lib, dev, M, N)
    ex_poly, tile_poly = tri_kernel_executed_flop(lib, dev, M, M)
    tri_exec = (n_kind[1] * ex_gram + n_kind[2] * ex_poly) / tri_launches if tri_launches else None
    achieved_exec = tri_exec / tri_ms / 1e9 if tri_ms else None
    norm_ms = per_kernel["normalize_cast"]
    norm_bytes = M * N * (4 + 2)  # float32 read once, bf16 written once
    failed = [] if res["parity"] == "ok" else ["mlp"]

    others = []
    if not args.no_others:
        for name in DEFAULT_OTHERS:
            torch.cuda.empty_cache()
            r = run_other(name, MIN_WARMUP, MIN_TIMED, lib, dev)
            others.append(r)
            if r["parity"] != "ok":
                failed.append(name)

    line = {
        "metric": "NS orthogonalize ms + TFLOP/s (% bf16 MFMA peak) at 4096x14336 bf16",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "zeros (power probe)" if zeros else "synthetic",
        "value_is": "effective throughput: the symmetric-halved FLOPs of five ordinary steps, 5 (3 m^2 n + m^3), over the "
        "measured time; the driver executes fewer (schedule below), so this is not MFMA utilisation",
        "pct_of_bf16_mfma_peak_nominal": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
        "pct_of_bf16_mfma_peak_executed": round(100.0 * f_exec / wall_ms / 1e9 / PEAK_BF16_TFLOPS, 2),
        "config": {
            "workload": f"newton_schulz, {NS_STEPS} steps ('simple' coefficients), one {M}x{N} float32 gradient "
            "(N(0,1e-3^2) with 1% entries at 50 sigma), bf16 MFMA kernels with fp32 accumulation, float32 result",
            "ms_median": res["ms_median"],
            "ms_min": res["ms_min"],
            "flops_counted": "symmetric-halved 5*(3 m^2 n + m^3): the count of five ordinary steps, whatever the schedule",
            "tflops_full_count": round(f_full / wall_ms / 1e9, 2),
            "schedule": "+".join(map(str, schedule)) + " (steps of one group share one Gram matrix)",
            "tflops_executed": round(f_exec / wall_ms / 1e9, 2),
            "pct_of_bf16_mfma_peak_executed": round(100.0 * f_exec / wall_ms / 1e9 / PEAK_BF16_TFLOPS, 2),
            "launches_per_call": {n: n_kind[i] // args.steps for i, n in enumerate(names)},
            "pct_of_bf16_mfma_peak": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
            "rel_fro_vs_fp32": res["rel_fro"],
            "tolerance": TOL,
            "parity": "ok" if not failed else "FAILED: " + ", ".join(failed),
            "kernel_ms": {k: (round(v, 4) if v is not None else None) for k, v in per_kernel.items()},
            "kernel_ms_note": "per launch group, from event pairs recorded around every group in a separate pass of the same "
            "steps; the brackets lengthen each figure by about 3 %, so their sum exceeds ms_per_step",
            "torch_bf16_path_ms": res.get("torch_bf16_path_ms"),
            "speedup_vs_torch": res.get("speedup_vs_torch"),
            "torch_bf16_path_rel_fro": res.get("torch_bf16_path_rel_fro"),
            "gemm_axpy_tflops": round(gemm_tflops, 1) if gemm_tflops else None,
            "gemm_axpy_traffic_bytes": GEMM_AXPY_TRAFFIC_BYTES if schedule == [3, 2] else None,
            "normalize_cast_gbps": round(norm_bytes / norm_ms / 1e6, 1) if norm_ms else None,
            "normalize_cast_pct_hbm_peak": round(100 * norm_bytes / norm_ms / 1e6 / PEAK_HBM_GBPS, 2) if norm_ms else None,
            "other_workloads": others,
        },
        "roofline": {
            "kernel": f"gemm_fast_kernel, lower-triangle mode ({tile_gram}^2 tiles for X X^T, {tile_poly}^2 for the m x m products; "
            f"{n_kind[1] // args.steps} + {n_kind[2] // args.steps} launches per call, sym-halved FLOP, average launch)",
            "bound": "mfma",
            "achieved": round(achieved, 2) if achieved else None,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4) if achieved else None,
            "frac_executed": round(achieved_exec / PEAK_BF16_TFLOPS, 4) if achieved_exec else None,
            "traffic": TRI_KERNEL_TRAFFIC_BYTES if (schedule == [3, 2] and tile_gram == 192 and tile_poly == 192) else None,
            "traffic_source": TRAFFIC_SOURCE,
            "avg_launch_ms": round(tri_ms, 4) if tri_ms else None,
        },
    }
    line["cpu_baseline"] = cpu_line
    print(json.dumps(line))
    if failed:
        sys.exit(1)


if __name__ == "__main__":
    main()
