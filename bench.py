#!/usr/bin/env python3
"""Headline benchmark: sparse spectral K(x, x) @ rhs, n = 100 000, k = 16, batch 8, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload headline|c1|...|ref_example]
                    [--variant auto|...] [--no-cpu-baseline] [--no-configs]

A step is one call of the operator over the whole batch with inputs resident in HBM.
Prints one JSON line: kernel-pair evaluations per second (``value``), the roofline of the
forward kernel against the MI355X fp32 peak (157.3 TFLOP/s, vector = matrix fp32), the same
figures for every other benchmark configuration (``configs``), the error of the default
(split-fp16) and of the fp32-MFMA contraction against a float64 evaluation of the whole output
(``roofline.error_vs_fp64``), and the CPU baseline (dense build-K-then-matmul in fp32 torch on
the host cores, bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3  # 256 CU x 256 flop/clk x 2.4 GHz; fp32 MFMA peak is the same figure

WORKLOADS = {
    # name: kernel, n, extent, batch, k, cutoff factor (x max lengthscale) or absolute, seed
    "headline": dict(kernel="spectral", n=100_000, extent=10_000.0, batch=8, k=16, cutoff_l=6.0, seed=1000,
                     label="spectral K@rhs n=100000 k=16 batch=8 x~U[0,10000) cutoff=6*l_max"),
    "c1": dict(kernel="rbf", n=4096, extent=100.0, batch=0, k=1, cutoff_abs=8.0, seed=1001,
               label="rbf K@rhs n=4096 k=1 l=sigma=1 cutoff=8"),
    "c2": dict(kernel="spectral", n=20_000, extent=2000.0, batch=4, k=16, cutoff_l=6.0, seed=1002,
               label="spectral K@rhs n=20000 k=16 batch=4 cutoff=6*l_max"),
    "c3": dict(kernel="spectral", n=50_000, extent=None, batch=2, k=8, cutoff_l=6.0, seed=1003, op="param_grad",
               label="spectral matmul_bwd n=50000 k=8 batch=2 x=cumsum(Exp(1)) cutoff=6*l_max"),
    "c3_rhs_grad": dict(kernel="spectral", n=50_000, extent=None, batch=2, k=8, cutoff_l=6.0, seed=1003,
                        label="spectral rhs gradient (K^T @ grad_out) n=50000 k=8 batch=2 x=cumsum(Exp(1))"),
    "c4": dict(kernel="spectral", n=100_000, extent=10_000.0, batch=16, k=4, cutoff_l=6.0, seed=1004, op="param_grad",
               label="spectral bilinear_derivative n=100000 d=4 batch=16 cutoff=6*l_max"),
    "c5": dict(kernel="spectral", n=1_000_000, extent=100_000.0, batch=8, k=32, cutoff_l=5.0, seed=1005,
               label="spectral K@rhs n=1000000 k=32 batch=8 cutoff=5*l_max"),
    # gradient at the headline's size with 8 vector columns (beyond the feature form's widths)
    "grad_c8": dict(kernel="spectral", n=100_000, extent=10_000.0, batch=8, k=8, cutoff_l=6.0, seed=1006, op="param_grad",
                    label="spectral bilinear_derivative n=100000 d=8 batch=8 cutoff=6*l_max"),
    # the reference's own benchmark recipe (examples/matmul.py:61-82 there)
    "ref_example": dict(kernel="rbf", n=65_536, extent=65_536 / 24.0, batch=1, k=64, cutoff_abs=10.0, seed=0,
                        label="rbf K@rhs n=65536 k=64 batch=1 x~U[0,n/24) cutoff=10 params=1+0.01*N(0,1)"),
}

# HBM bytes per launch of the headline kernel, from the FETCH_SIZE / WRITE_SIZE counter runs
# summarised in the file named here (an offline rocprofv3 --pmc run, not measured by this script).
# Untimed continuous launches before a timed region, in milliseconds (clock ramp of the GPU).
SPIN_UP_MS = 100.0

TRAFFIC_SOURCE = "profiles/fwd_table_f16_grouped_headline_counters.md"
MEASURED_TRAFFIC_BYTES = {"headline": 58609869}

# Share of the kernel's cycles in which the SIMDs' VALU is busy (SQ_ACTIVE_INST_VALU x 4 / SIMD
# cycles), from the offline counter runs summarised under profiles/ (not measured by this script).
VALU_BUSY = {
    "headline": (0.75, "profiles/fwd_table_f16_grouped_headline_counters.md"),
    "headline_fp32": (0.46, "profiles/fwd_table_f32_grouped_headline_profile.md"),
    "c1": (0.11, "profiles/fwd_table_f16_midsize_c1_c2_c3_profile.md"),
    "c2": (0.46, "profiles/fwd_table_f16_midsize_c1_c2_c3_profile.md"),
    "c3": (0.45, "profiles/param_grad_partial_c3_and_wide_vectors_profile.md"),
    "c3_rhs_grad": (0.47, "profiles/fwd_table_f16_midsize_c1_c2_c3_profile.md"),
    "c4": (0.73, "profiles/param_grad_features_c4_profile.md"),
    "c5": (0.95, "profiles/forward_c5_and_reference_recipe_profile.md"),
    "grad_c8": (0.62, "profiles/param_grad_partial_c3_and_wide_vectors_profile.md"),
    "ref_example": (0.43, "profiles/forward_c5_and_reference_recipe_profile.md"),
}


def pipe_of(kernel_description: str) -> str:
    """Which pipes do the work of the kernel the library says it launches."""
    if "fwd_valu" in kernel_description:
        return "valu"
    if "f32" in kernel_description or "param_grad_partial" in kernel_description:
        return "valu+mfma_f32"
    return "valu+mfma_f16"

FLOPS_PER_PAIR = {"rbf": lambda k: 5 + 2 * k, "spectral": lambda k: 8 + 2 * k,
                  "locally_periodic": lambda k: 10 + 2 * k}
GRAD_FLOPS_PER_PAIR = {"rbf": lambda c: 6 + 2 * c + 2 * 2, "spectral": lambda c: 14 + 2 * c + 2 * 3}


def make_workload(name: str, batch_override=None):
    """Seeded CPU generation (so the GPU run and the CPU baseline see identical bits)."""
    import torch

    w = dict(WORKLOADS[name])
    if batch_override is not None:
        w["batch"] = batch_override
        w["label"] += f" [batch overridden to {batch_override}]"
    g = torch.Generator().manual_seed(w["seed"])
    n, batch = w["n"], w["batch"]
    if w["extent"] is None:  # irregular grid: cumulative sum of Exp(1) gaps
        x = torch.cumsum(-torch.log1p(-torch.rand(n, generator=g)), dim=0)
    else:
        x = torch.sort(torch.rand(n, generator=g) * w["extent"])[0]
    bshape = (batch,) if batch else ()
    u = lambda lo, hi: lo + (hi - lo) * torch.rand(bshape, generator=g)
    if name == "ref_example":
        params = 1.0 + 0.01 * torch.randn(*bshape, 2, generator=g)
    elif w["kernel"] == "spectral":
        params = torch.stack([u(0.5, 2.0), u(0.05, 0.5), u(0.5, 2.0)], dim=-1)
    elif w["kernel"] == "locally_periodic":
        params = torch.stack([u(0.5, 2.0), u(0.5, 2.0), u(0.5, 2.0), u(0.5, 2.0)], dim=-1)
    else:
        params = torch.stack([torch.ones(bshape), torch.ones(bshape)], dim=-1)
    rhs = torch.randn(n, w["k"], generator=g)
    if name == "ref_example":
        rhs = rhs / rhs.norm(dim=0, keepdim=True)
    cutoff = w["cutoff_abs"] if "cutoff_abs" in w else w["cutoff_l"] * float(params[..., 0].max())
    return w, x, params.float(), rhs, cutoff


class Prepared:
    """One workload resident on the GPU, ready to be called."""

    def __init__(self, name, device, batch_override=None, variant="auto", rows_per_wave=0, col_splits=0,
                 tail_balance=True, group_tail=None, group_tail_halves=None):
        import torch

        from kernel_matmul_amd.compile import load_native
        from kernel_matmul_amd.configurations import BilinearDerivativeConfiguration, MatmulSingleConfiguration
        from kernel_matmul_amd.ranges import make_ranges

        self.name = name
        self.w, self.x_cpu, self.params_cpu, self.rhs_cpu, self.cutoff = make_workload(name, batch_override)
        w = self.w
        n, k, batch = w["n"], w["k"], w["batch"]
        bshape = (batch,) if batch else ()
        self.start_cpu, self.end_cpu = make_ranges(self.cutoff, self.x_cpu)  # symmetric pattern, block 128
        row_blocks = self.start_cpu.shape[-1]
        rows_in_block = torch.clamp(n - 128 * torch.arange(row_blocks), max=128)
        self.pairs = int((rows_in_block * (self.end_cpu - self.start_cpu)).sum()) * max(batch, 1)
        self.is_grad = w.get("op") == "param_grad"
        self.flops_per_pair = (GRAD_FLOPS_PER_PAIR if self.is_grad else FLOPS_PER_PAIR)[w["kernel"]](k)

        x = self.x_cpu.to(device)
        rhs = self.rhs_cpu.to(device)
        self.params = self.params_cpu.to(device)
        start, end = self.start_cpu.to(device), self.end_cpu.to(device)
        # batch items share x, rhs and the pattern (stride-0 views), as KernelMatmulLinearOperator passes them
        xb = x.expand(*bshape, n)
        rhsb = rhs.expand(*bshape, n, k)
        startb = start.expand(*bshape, row_blocks)
        endb = end.expand(*bshape, row_blocks)
        if name == "c3_rhs_grad":
            # d/d rhs of sum(grad_out * (K @ rhs)) = K^T @ grad_out: the forward kernel on the
            # (symmetric) pattern with a per-batch-item grad_out in place of rhs
            g2 = torch.Generator().manual_seed(w["seed"] + 60)
            rhsb = torch.randn(*bshape, n, k, generator=g2).to(device)
        self.args = (xb, xb, rhsb, self.params, startb, endb)
        defines = MatmulSingleConfiguration(w["kernel"]).make_config(self.args)
        if variant != "auto":
            defines["MATMUL_VARIANT"] = variant
        if rows_per_wave:
            defines["MATMUL_ROWS_PER_WAVE"] = rows_per_wave
        if col_splits:
            defines["MATMUL_COL_BLOCKS"] = col_splits
        if not tail_balance:
            defines["MATMUL_TAIL_BALANCE"] = 0
        if group_tail is not None:
            defines["MATMUL_GROUP_TAIL"] = group_tail
            if group_tail_halves is not None:
                defines["MATMUL_GROUP_TAIL_HALVES"] = group_tail_halves
        self.op = load_native("matmul", defines)
        self.kernel = self.op.describe(*self.args)
        if self.is_grad:
            g2 = torch.Generator().manual_seed(w["seed"] + 50)
            left = torch.randn(n, k, generator=g2).to(device).expand(*bshape, n, k)
            self.args = (xb, xb, left, rhsb, self.params, startb, endb)
            self.op = load_native("bilinear_derivative",
                                  BilinearDerivativeConfiguration(w["kernel"]).make_config(self.args))
            self.kernel = self.op.describe(*self.args)

    def call(self):
        return self.op.call(*self.args)

    def measure(self, steps, warmup, spin_up_ms=SPIN_UP_MS):
        """Times `steps` calls twice and returns a dict of milliseconds per call.

        After the `warmup` calls the same call is repeated for `spin_up_ms` more (untimed): the
        GPU raises its clocks over the first tens of milliseconds of continuous work, and launches
        in that phase take up to 20 % longer than in steady state.

        Timed region: the calls issued back to back between two synchronisations, with one event
        before the first and one after the last launch on the launch stream (`wall_ms`,
        `stream_ms`).  Second pass: the same calls with an event pair around every launch
        (`kernel_ms`, `kernel_ms_median`): the duration of one launch on its own, the figure a
        kernel trace reports.
        """
        import torch

        out = None
        for _ in range(warmup):
            out = self.call()
        torch.cuda.synchronize()
        t_spin = time.perf_counter()
        while (time.perf_counter() - t_spin) * 1e3 < spin_up_ms:
            for _ in range(20):
                out = self.call()
            torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        first.record()
        for _ in range(steps):
            out = self.call()
        last.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()

        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                  for _ in range(steps)]
        for e0, e1 in events:
            e0.record()
            out = self.call()
            e1.record()
        torch.cuda.synchronize()
        kernel_ms = sorted(e0.elapsed_time(e1) for e0, e1 in events)
        return {
            "wall_ms": (t1 - t0) * 1e3 / steps,
            "stream_ms": first.elapsed_time(last) / steps,
            "kernel_ms": sum(kernel_ms) / len(kernel_ms),
            "kernel_ms_median": kernel_ms[len(kernel_ms) // 2],
            "out": out,
        }

    def summary(self, steps, warmup):
        t = self.measure(steps, warmup)
        flops = self.pairs * self.flops_per_pair
        return {
            "workload": self.w["label"],
            "kernel": self.kernel,
            "pairs_per_call": self.pairs,
            "flops_per_pair": self.flops_per_pair,
            "kernel_ms": t["kernel_ms"],
            "kernel_ms_median": t["kernel_ms_median"],
            "back_to_back_ms_per_call": t["stream_ms"],
            "wall_ms_per_call": t["wall_ms"],
            "pairs_per_s_kernel": self.pairs / (t["kernel_ms"] * 1e-3),
            "pairs_per_s_wall": self.pairs / (t["wall_ms"] * 1e-3),
            # nominal flops (direct evaluation, fp32 contraction) per second over the fp32 peak: a
            # normalised throughput, above 1 where the contraction runs on the fp16 matrix pipe
            "algorithmic_frac_vs_fp32_peak": flops / (t["kernel_ms"] * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
            "algorithmic_frac_vs_fp32_peak_back_to_back": flops / (t["stream_ms"] * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
            "pipe": pipe_of(self.kernel),
            "valu_busy": VALU_BUSY.get(self.name, (None, None))[0],
            "valu_busy_source": VALU_BUSY.get(self.name, (None, None))[1],
        }


def time_index_and_ranges(device, steps=50):
    """The rest of benchmark configuration 5: kernel rows at 4096 random (batch, row, column) indices
    and the symmetric range computation at n = 10^6, both on the GPU.  Latency-bound operations:
    reported as time per call only."""
    import torch

    from kernel_matmul_amd.compile import load_native
    from kernel_matmul_amd.configurations import IndexConfiguration
    from kernel_matmul_amd.ranges import make_ranges

    w, x_cpu, params_cpu, _, cutoff = make_workload("c5")
    n, batch = w["n"], w["batch"]
    x = x_cpu.to(device)
    make_ranges(cutoff, x, check_sorted=False)
    torch.cuda.synchronize()

    def timed(call):
        for _ in range(5):
            call()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            call()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    ranges_ms = timed(lambda: make_ranges(cutoff, x, check_sorted=False))
    start, end = make_ranges(cutoff, x, check_sorted=False)
    g = torch.Generator().manual_seed(w["seed"] + 70)
    rows = torch.randint(0, n, (4096,), generator=g)
    cols = torch.clamp(rows + torch.randint(-600, 600, (4096,), generator=g), 0, n - 1)
    bi = torch.randint(0, batch, (4096,), generator=g)
    to = lambda t: t.to(torch.int32).to(device)
    blocks = start.shape[-1]
    args = (x.expand(batch, n), x.expand(batch, n), params_cpu.to(device), start.expand(batch, blocks),
            end.expand(batch, blocks), (to(bi),), to(rows), to(cols))
    op = load_native("index", IndexConfiguration(w["kernel"]).make_config(args))
    index_ms = timed(lambda: op.call(*args))
    return {
        "workload": "spectral, n=1000000, batch=8: index lookup of 4096 random (batch, row, column) entries; "
                    "symmetric ranges of all 7813 row blocks on the GPU",
        "index_ms_per_call": index_ms,
        "ranges_ms_per_call": ranges_ms,
        "note": "latency-bound operations, wall time per call from Python (launch and argument marshalling "
                "included); no roofline fraction is meaningful here",
    }


def full_output_fp64(p: Prepared):
    """float64 K @ rhs over the whole pattern of a forward workload, one row block at a time."""
    import numpy as np

    from oracle import kernels as oracle

    x = p.x_cpu.numpy()
    rhs = p.rhs_cpu.double().numpy()
    params = p.params_cpu.numpy().reshape(-1, p.params_cpu.shape[-1])
    start, end = p.start_cpu.numpy(), p.end_cpu.numpy()
    n, nb = x.shape[0], params.shape[0]
    out = np.zeros((nb, n, rhs.shape[-1]))
    for blk in range(len(start)):
        r0, r1 = blk * 128, min(blk * 128 + 128, n)
        s, e = int(start[blk]), min(int(end[blk]), n)
        if s < e:
            kb = oracle.kernel_matrix(p.w["kernel"], np.broadcast_to(x[r0:r1], (nb, r1 - r0)),
                                      np.broadcast_to(x[s:e], (nb, e - s)), params)
            out[:, r0:r1] = kb @ rhs[s:e]
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spin-up-ms", type=float, default=SPIN_UP_MS,
                    help="untimed continuous launches after the warm-up steps (the GPU's clock ramp)")
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS))
    ap.add_argument("--variant", default="auto", choices=["auto", "block", "mfma_f32", "mfma_f32_direct", "mfma_f16", "mfma_f16_direct", "valu"])
    ap.add_argument("--rows-per-wave", type=int, default=0)
    ap.add_argument("--col-splits", type=int, default=0)
    ap.add_argument("--batch", type=int, default=None, help="override the number of batch items")
    ap.add_argument("--no-tail-balance", action="store_true")
    ap.add_argument("--group-tail", type=int, default=None,
                    help="table kernel: grouped launch with this many column-split items per XCD")
    ap.add_argument("--group-tail-halves", type=int, default=None,
                    help="with --group-tail: how many of those items also run as two halves of 64 rows")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the host-side legs: the CPU baseline and the float64 error figures")
    ap.add_argument("--no-configs", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB elementwise add-scalar (a copy-like kernel of known traffic "
                         "against which FETCH_SIZE / WRITE_SIZE counters are scaled)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus must be 1 "
              "(the path has no collective or multi-GPU part).", file=sys.stderr)
        return 2

    import torch

    from kernel_matmul_amd import _native

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    _native.load_library()  # fail loudly if the HIP library is missing
    device = torch.device("cuda:0")

    main_run = Prepared(args.workload, device, args.batch, args.variant, args.rows_per_wave, args.col_splits,
                        not args.no_tail_balance, args.group_tail, args.group_tail_halves)
    w = main_run.w
    n, batch = w["n"], w["batch"]

    for _ in range(args.warmup):
        out = main_run.call()
    torch.cuda.synchronize()
    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 1.0, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    default_run = args.workload == "headline" and args.batch is None and args.variant in ("auto", "mfma_f16")
    traffic = MEASURED_TRAFFIC_BYTES["headline"] if default_run else None

    # The same steps right after the warm-up, before the GPU has raised its clocks.
    cold = main_run.measure(args.steps, 0, 0.0)
    # Whole-step wall time of the timed region and, on the launch stream, the event time over the
    # region and around single launches.
    timing = main_run.measure(args.steps, 0, args.spin_up_ms)
    ms_per_step, out = timing["wall_ms"], timing["out"]
    kernel_ms_avg, kernel_ms_med = timing["kernel_ms"], timing["kernel_ms_median"]
    pairs, flops_per_pair = main_run.pairs, main_run.flops_per_pair
    value = pairs / (ms_per_step * 1e-3)
    achieved_tflops = pairs * flops_per_pair / (kernel_ms_avg * 1e-3) / 1e12
    back_to_back_tflops = pairs * flops_per_pair / (timing["stream_ms"] * 1e-3) / 1e12


    result = {
        "metric": "kernel-pair evaluations/s (sparse spectral K@rhs, n=100k, k=16, 1 MI355X)",
        "value": value,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "spin_up_ms": args.spin_up_ms,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 in/out, K evaluated in f32 on the VALU; contraction: split-fp16 MFMA (hi+lo, 22 bits per "
                 "factor) with f32 accumulation (roofline.fp32_mfma_variant: the same with every product in f32)"
                 if args.variant in ("auto", "mfma_f16", "mfma_f16_direct", "block") else "f32",
        "data": "synthetic",
        "config": {
            "workload": w["label"],
            "pairs_per_step": pairs,
            "flops_per_pair": flops_per_pair,
            "variant": main_run.op.defines.get("MATMUL_VARIANT", "auto"),
            "seed": w["seed"],
        },
        "roofline": {
            "bound": "valu",
            "kernel": main_run.kernel,
            "achieved": achieved_tflops,
            "peak": PEAK_FP32_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved_tflops / PEAK_FP32_TFLOPS,
            "traffic": traffic,
            "traffic_source": TRAFFIC_SOURCE + " (offline counter run, not measured by this run)" if traffic else None,
            "kernel_ms_avg": kernel_ms_avg,
            "kernel_ms_median": kernel_ms_med,
            "pairs_per_s_kernel": pairs / (kernel_ms_avg * 1e-3),
            "timing": "achieved / frac: one launch on its own (event pair around every launch, second pass "
                      "of the same steps) - the duration a kernel trace reports; back_to_back: events around "
                      "the whole timed region / steps, launches queued without events in between",
            "back_to_back": {
                "kernel_ms": timing["stream_ms"],
                "achieved": back_to_back_tflops,
                "frac": back_to_back_tflops / PEAK_FP32_TFLOPS,
            },
            "cold": {
                "what": "the same steps timed right after --warmup, without the spin-up launches",
                "ms_per_step": cold["wall_ms"],
                "pairs_per_s": pairs / (cold["wall_ms"] * 1e-3),
                "kernel_ms_avg": cold["kernel_ms"],
                "frac": pairs * flops_per_pair / (cold["kernel_ms"] * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
            },
            "pipe": pipe_of(main_run.kernel),
            "valu_busy": VALU_BUSY["headline"][0] if default_run else None,
            "valu_busy_source": VALU_BUSY["headline"][1] if default_run else None,
            # what the launched kernel executes per wavefront-wide group of 64 pairs (SQ_INSTS_VALU and
            # SQ_INSTS_MFMA of the same counter runs over the 5.14 M groups of a launch)
            "executed_per_64_pairs": {"valu_instructions": 8.1, "mfma_f32_16x16x32_f16": 0.75}
                                     if default_run else None,
            "achieved_is": "nominal flops per pair (8 + 2k: direct evaluation, fp32 contraction) x pairs / kernel "
                           "time; the kernel launched executes fewer VALU operations per pair (separable exponent, "
                           "tabulated phases) and contracts on the matrix pipe named in `pipe`",
            "note": "bound by VALU issue (kernel evaluation in fp32 + hi/lo split + MFMA issue), priced against "
                    "the fp32 peak (157.3 TFLOP/s vector == fp32 MFMA); flops = pairs * (8 + 2k), one "
                    "transcendental counted as 1.  The contraction itself runs as split-fp16 MFMAs, so frac is "
                    "a figure of merit against the fp32 roofline, not a utilisation of one pipe",
        },
    }

    if default_run:
        # The same workload with the contraction as a true fp32 MFMA (v_mfma_f32_16x16x4_f32): K
        # evaluated in fp32 on the VALU, every product and sum of the contraction in fp32.
        f32_run = Prepared("headline", device, variant="mfma_f32")
        f32_timing = f32_run.measure(max(args.steps // 2, 5), 2)
        f32_ms, f32_out = f32_timing["kernel_ms"], f32_timing["out"]
        result["roofline"]["fp32_mfma_variant"] = {
            "kernel": f32_run.kernel,
            "pipe": pipe_of(f32_run.kernel),
            "valu_busy": VALU_BUSY["headline_fp32"][0],
            "mfma_busy": 0.395,
            "busy_source": VALU_BUSY["headline_fp32"][1] + " (VALU and fp32-MFMA cycles are disjoint on gfx950: "
                           "together 86 % of the kernel's cycles at batch 8, 95 % at batch 64)",
            "kernel_ms": f32_ms,
            "frac": pairs * flops_per_pair / (f32_ms * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
            "back_to_back_kernel_ms": f32_timing["stream_ms"],
            "back_to_back_frac": pairs * flops_per_pair / (f32_timing["stream_ms"] * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
        }
    else:
        f32_out = None

    if not args.no_configs and default_run:
        configs = {}
        for name in ("c1", "c2", "c3", "c3_rhs_grad", "c4", "c5", "ref_example"):
            run = Prepared(name, device)
            # (launches of tens of microseconds: enough steps that a few slow ones do not carry the mean)
            configs[name] = run.summary(steps={"c5": 50, "c4": 100}.get(name, 200), warmup=5)
            del run
            torch.cuda.empty_cache()
        configs["c5_index_and_ranges"] = time_index_and_ranges(device)
        result["configs"] = configs

    if not args.no_cpu_baseline and not main_run.is_grad:
        import numpy as np

        from oracle import dense_cpu

        if default_run:
            # Error of both contractions over the whole output against float64.
            expected = full_output_fp64(main_run)
            scale = np.abs(expected).max()
            errors = {}
            for label, tensor in (("auto", out), ("mfma_f32", f32_out)):
                err = np.abs(tensor.cpu().double().numpy() - expected)
                errors[label] = {
                    "max_abs": float(err.max()),
                    "max_abs_over_output_scale": float(err.max() / scale),
                    "max_rel_where_abs_expected_ge_1e-3": float((err / np.maximum(np.abs(expected), 1e-3)).max()),
                    "rms": float(np.sqrt((err * err).mean())),
                }
            errors["output_scale_max_abs"] = float(scale)
            errors["tolerance"] = "rtol 1e-4 / atol 1e-5 (tests), both variants within it"
            result["roofline"]["error_vs_fp64"] = errors
            del expected

        x_cpu, rhs_cpu, params_cpu = main_run.x_cpu, main_run.rhs_cpu, main_run.params_cpu
        p0 = params_cpu[0] if batch else params_cpu
        sec, in_band, dense_pairs, slabs, rows = dense_cpu.time_masked_matmul(
            w["kernel"], x_cpu, x_cpu, rhs_cpu, p0, main_run.start_cpu, main_run.end_cpu, args.cpu_seconds)
        got = (out[0] if batch else out)[: rows.shape[0]].cpu()
        err = (got - rows).abs().max().item()
        result["cpu_baseline"] = {
            "value": in_band / sec,
            "unit": "pairs/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"dense fp32 torch build-K-then-matmul of the first {rows.shape[0]} rows "
                      f"({slabs} slabs of 1024 rows x {n} cols) of batch item 0; "
                      f"{sec:.1f} s; dense pairs/s {dense_pairs / sec:.3e}; "
                      f"max |gpu - cpu| on these rows {err:.2e}; os.cpu_count()={os.cpu_count()}",
        }

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
