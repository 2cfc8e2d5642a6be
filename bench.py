#!/usr/bin/env python3
"""Headline benchmark: sparse spectral K(x, x) @ rhs, n = 100 000, k = 16, batch 8, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload headline|c1|c2|c5]
                    [--variant auto|mfma|valu] [--no-cpu-baseline]

A step is one call of the matmul operator over the whole batch with inputs resident in HBM.
Prints one JSON line: kernel-pair evaluations per second (``value``), the roofline of the
forward kernel against the MI355X fp32 peak (157.3 TFLOP/s, vector = matrix fp32), and the
CPU baseline (dense build-K-then-matmul in fp32 torch on the host cores, bounded sample).
"""
from __future__ import annotations

import argparse
import json
import math
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
    "c4": dict(kernel="spectral", n=100_000, extent=10_000.0, batch=16, k=4, cutoff_l=6.0, seed=1004, op="param_grad",
               label="spectral bilinear_derivative n=100000 d=4 batch=16 cutoff=6*l_max"),
    "c5": dict(kernel="spectral", n=1_000_000, extent=100_000.0, batch=8, k=32, cutoff_l=5.0, seed=1005,
               label="spectral K@rhs n=1000000 k=32 batch=8 cutoff=5*l_max"),
}

# (FETCH_SIZE 3543.6 KiB x 2.00 + WRITE_SIZE 50000.0 KiB x 1.00) x 1024
MEASURED_TRAFFIC_BYTES = {"headline": 58763674}

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
    if w["kernel"] == "spectral":
        params = torch.stack([u(0.5, 2.0), u(0.05, 0.5), u(0.5, 2.0)], dim=-1)
    else:
        params = torch.stack([torch.ones(bshape), torch.ones(bshape)], dim=-1)
    rhs = torch.randn(n, w["k"], generator=g)
    cutoff = w["cutoff_abs"] if "cutoff_abs" in w else w["cutoff_l"] * float(params[..., 0].max())
    return w, x, params.float(), rhs, cutoff


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS))
    ap.add_argument("--variant", default="auto", choices=["auto", "block", "mfma_f32", "mfma_f16", "mfma_f16_direct", "valu"])
    ap.add_argument("--rows-per-wave", type=int, default=0)
    ap.add_argument("--col-splits", type=int, default=0)
    ap.add_argument("--batch", type=int, default=None, help="override the number of batch items")
    ap.add_argument("--no-tail-balance", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    from kernel_matmul_amd.compile import load_native
    from kernel_matmul_amd.configurations import MatmulSingleConfiguration
    from kernel_matmul_amd.ranges import make_ranges

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    _native.load_library()  # fail loudly if the HIP library is missing
    device = torch.device("cuda:0")

    w, x_cpu, params_cpu, rhs_cpu, cutoff = make_workload(args.workload, args.batch)
    n, k, batch = w["n"], w["k"], w["batch"]
    bshape = (batch,) if batch else ()
    start_cpu, end_cpu = make_ranges(cutoff, x_cpu)  # symmetric pattern, block 128
    row_blocks = start_cpu.shape[-1]
    rows_in_block = torch.clamp(n - 128 * torch.arange(row_blocks), max=128)
    pairs_per_item = int((rows_in_block * (end_cpu - start_cpu)).sum())
    pairs = pairs_per_item * max(batch, 1)
    is_grad = w.get("op") == "param_grad"
    flops_per_pair = (GRAD_FLOPS_PER_PAIR if is_grad else FLOPS_PER_PAIR)[w["kernel"]](k)

    x = x_cpu.to(device)
    rhs = rhs_cpu.to(device)
    params = params_cpu.to(device)
    start, end = start_cpu.to(device), end_cpu.to(device)
    # batch items share x, rhs and the pattern (stride-0 views), as KernelMatmulLinearOperator passes them
    xb = x.expand(*bshape, n)
    rhsb = rhs.expand(*bshape, n, k)
    startb = start.expand(*bshape, row_blocks)
    endb = end.expand(*bshape, row_blocks)
    op_args = (xb, xb, rhsb, params, startb, endb)

    defines = MatmulSingleConfiguration(w["kernel"]).make_config(op_args)
    if args.variant != "auto":
        defines["MATMUL_VARIANT"] = args.variant
    if args.rows_per_wave:
        defines["MATMUL_ROWS_PER_WAVE"] = args.rows_per_wave
    if args.col_splits:
        defines["MATMUL_COL_BLOCKS"] = args.col_splits
    if args.no_tail_balance:
        defines["MATMUL_TAIL_BALANCE"] = 0
    op = load_native("matmul", defines)
    if is_grad:
        from kernel_matmul_amd.configurations import BilinearDerivativeConfiguration

        g2 = torch.Generator().manual_seed(w["seed"] + 50)
        left = torch.randn(n, k, generator=g2).to(device).expand(*bshape, n, k)
        op_args = (xb, xb, left, rhsb, params, startb, endb)
        op = load_native("bilinear_derivative",
                         BilinearDerivativeConfiguration(w["kernel"]).make_config(op_args))

    for _ in range(args.warmup):
        out = op.call(*op_args)
    torch.cuda.synchronize()
    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 1.0, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # Whole-step wall time and, on the launch stream, per-launch event time of the kernel.
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e0, e1 in events:
        e0.record()
        out = op.call(*op_args)
        e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernel_ms = sorted(e0.elapsed_time(e1) for e0, e1 in events)
    kernel_ms_avg = sum(kernel_ms) / len(kernel_ms)
    kernel_ms_med = kernel_ms[len(kernel_ms) // 2]

    value = pairs / (ms_per_step * 1e-3)
    achieved_tflops = pairs * flops_per_pair / (kernel_ms_avg * 1e-3) / 1e12

    # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
    # profiles/fwd_table_f16_headline_counters.md (only measured for the default headline run).
    traffic = None
    if args.workload == "headline" and args.batch is None and args.variant in ("auto", "mfma_f16"):
        traffic = MEASURED_TRAFFIC_BYTES["headline"]

    # Kernel the launch table picks for this workload / variant: column tables (spectral in
    # phase-split form) for rbf / spectral with at most 16 rhs columns, the shared-operand kernel
    # for large rbf / locally periodic problems, direct evaluation otherwise.
    row_block_items = ((n + 127) // 128) * max(batch, 1)
    table = w["kernel"] in ("spectral", "rbf") and k <= 16
    shared = w["kernel"] != "spectral" and k <= 16 and row_block_items >= 4096
    auto_kernel = "km::fwd_block" if shared else ("km::fwd_table_f16" if table else "km::fwd_mfma_f16")
    kernel_name = "km::param_grad_partial" if is_grad else {
        "auto": auto_kernel,
        "mfma_f16": "km::fwd_table_f16" if table else "km::fwd_mfma_f16",
        "mfma_f16_direct": "km::fwd_mfma_f16", "block": "km::fwd_block",
        "mfma_f32": "km::fwd_mfma_f32", "valu": "km::fwd_valu"}[args.variant]

    result = {
        "metric": "kernel-pair evaluations/s (sparse spectral K@rhs, n=100k, k=16, 1 MI355X)",
        "value": value,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": w["label"],
            "pairs_per_step": pairs,
            "flops_per_pair": flops_per_pair,
            "variant": op.defines.get("MATMUL_VARIANT", "auto (split-fp16 MFMA)"),
            "seed": w["seed"],
        },
        "roofline": {
            "bound": "mfma",
            "kernel": kernel_name,
            "achieved": achieved_tflops,
            "peak": PEAK_FP32_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved_tflops / PEAK_FP32_TFLOPS,
            "traffic": traffic,
            "kernel_ms_avg": kernel_ms_avg,
            "kernel_ms_median": kernel_ms_med,
            "pairs_per_s_kernel": pairs / (kernel_ms_avg * 1e-3),
            "note": "priced against the fp32 peak (157.3 TFLOP/s vector == fp32 MFMA): K is evaluated in "
                    "fp32 on the VALU, the contraction runs as split-fp16 MFMAs with fp32 accumulation; "
                    "flops = pairs * (8 + 2k), one transcendental counted as 1",
        },
    }

    if not args.no_cpu_baseline and not is_grad:
        from oracle import dense_cpu

        p0 = params_cpu[0] if batch else params_cpu
        sec, in_band, dense_pairs, slabs, rows = dense_cpu.time_masked_matmul(
            w["kernel"], x_cpu, x_cpu, rhs_cpu, p0, start_cpu, end_cpu, args.cpu_seconds)
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
