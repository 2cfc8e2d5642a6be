#!/usr/bin/env python3
"""Writes tests/golden/ranges_golden.npz from the reference's own range builder.

The vectors come from `oracle/_ref/km_ranges_ref.so`, i.e. the reference's
native/ranges/ranges.cpp compiled unmodified by oracle/build_ref.sh.  Only inputs and
outputs are stored.  Run in a container that has the reference tree:

    sh oracle/build_ref.sh && python tests/golden/make_ranges_golden.py

Cases: block sizes 1, 3 and 128; random, duplicated, gapped and offset grids; cutoffs from 0
to larger than the data extent; aligned and unaligned; sizes below, at and above one block.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle", "_ref"))
import km_ranges_ref as ref  # noqa: E402


def grid(rng, batch, n, kind):
    if kind == "uniform":
        x = rng.random((batch, n)) * 10
    elif kind == "dup":
        x = rng.integers(0, max(n // 3, 2), (batch, n)) / 4.0
    elif kind == "gap":
        x = rng.random((batch, n)) * 10
        x[:, n // 3:] += 20
    elif kind == "wide":
        x = rng.random((batch, n)) * 1000
    elif kind == "cumexp":
        x = np.cumsum(rng.exponential(1.0, (batch, n)), axis=1)
    else:
        raise ValueError(kind)
    return np.sort(x.astype(np.float32), axis=1)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    case = 0
    specs = []
    for bs in (1, 3, 128):
        for kind in ("uniform", "dup", "gap", "wide", "cumexp"):
            for (n1, n2) in ((50, 55), (129, 130), (600, 800), (128, 128), (5, 300), (1000, 77)):
                for cutoff in (0.0, 0.1, 1.0, 11.0, 2000.0):
                    if rng.random() < 0.82:  # keep the fixture small
                        continue
                    specs.append((bs, kind, n1, n2, cutoff))
    for bs, kind, n1, n2, cutoff in specs:
        batch = int(rng.integers(1, 4))
        x1 = grid(rng, batch, n1, kind)
        x2 = grid(rng, batch, n2, kind) + np.float32(rng.choice([0.0, -1.0, 1.5]))
        for align in (False, True):
            s, e = ref.make_ranges(torch.from_numpy(x1), torch.from_numpy(x2), cutoff, bs, align)
            key = f"asym{case:04d}"
            out[key + "_x1"], out[key + "_x2"] = x1, x2
            out[key + "_meta"] = np.array([cutoff, bs, int(align)], dtype=np.float64)
            out[key + "_start"], out[key + "_end"] = s.numpy(), e.numpy()
            if align:
                st, et = ref.transpose_ranges(s, e, n1, n2, bs)
                out[key + "_start_t"], out[key + "_end_t"] = st.numpy(), et.numpy()
            case += 1
        s, e = ref.make_ranges_symmetric(torch.from_numpy(x1), cutoff, bs)
        key = f"sym{case:04d}"
        out[key + "_x"] = x1
        out[key + "_meta"] = np.array([cutoff, bs], dtype=np.float64)
        out[key + "_start"], out[key + "_end"] = s.numpy(), e.numpy()
        case += 1
    # larger block-128 grids shaped like the benchmark workloads
    for n, extent, cutoff in ((4096, 100.0, 8.0), (20000, 2000.0, 9.0), (30000, None, 7.5)):
        if extent is None:
            x = np.cumsum(rng.exponential(1.0, (1, n)), axis=1).astype(np.float32)
        else:
            x = np.sort((rng.random((1, n)) * extent).astype(np.float32), axis=1)
        s, e = ref.make_ranges_symmetric(torch.from_numpy(x), cutoff, 128)
        key = f"sym{case:04d}"
        out[key + "_x"] = x
        out[key + "_meta"] = np.array([cutoff, 128], dtype=np.float64)
        out[key + "_start"], out[key + "_end"] = s.numpy(), e.numpy()
        case += 1
    path = os.path.join(HERE, "ranges_golden.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {case} cases, {os.path.getsize(path) / 1024:.0f} KiB -> {path}")


if __name__ == "__main__":
    main()
