"""CPU baseline: the reference's dense build-K-then-matmul check path in fp32 torch.

TEST / BENCHMARK INFRASTRUCTURE: imported by bench.py's cpu_baseline leg and by tests only.

Restates what the reference's tests do to obtain their expected result: build the dense kernel
matrix, keep rows [128 i, 128 (i+1)) x columns [start_i, end_i) and zero the rest
(tests/conftest.py:179-249), then ``masked_K @ rhs`` (tests/native/test_matmul.py:28).
GPyTorch is replaced by the closed forms it evaluates (see oracle/kernels.py).  For large n
the matrix is built in slabs of whole row blocks x all n columns: identical arithmetic,
bounded memory.
"""
from __future__ import annotations

import math
import time

import torch

BLOCK_SIZE = 128


def dense_kernel_rows(kernel_type: str, x1_rows: torch.Tensor, x2: torch.Tensor,
                      params: torch.Tensor) -> torch.Tensor:
    """K[rows, n] in fp32 for one batch item (params is 1-D)."""
    d = x1_rows[:, None] - x2[None, :]
    if kernel_type == "rbf":
        l, s = params[0], params[1]
        return s * torch.exp(-(d * d) / (2 * l * l))
    if kernel_type == "spectral":
        l, f, s = params[0], params[1], params[2]
        return s * torch.exp(-(d * d) / (2 * l * l)) * torch.cos((2 * math.pi) * f * d)
    if kernel_type == "locally_periodic":
        l, lp, period, s = params[0], params[1], params[2], params[3]
        sn = torch.sin(math.pi * d / period)
        return s * torch.exp(-(d * d) / (2 * l * l) - (2 / lp) * sn * sn)
    raise ValueError(kernel_type)


def masked_matmul_slab(kernel_type, x1, x2, rhs, params, start, end, block_from: int,
                       block_to: int) -> torch.Tensor:
    """Rows of row blocks [block_from, block_to) of masked K @ rhs for one batch item."""
    m = x1.shape[0]
    row_from = block_from * BLOCK_SIZE
    row_to = min(block_to * BLOCK_SIZE, m)
    k = dense_kernel_rows(kernel_type, x1[row_from:row_to], x2, params)
    cols = torch.arange(x2.shape[0])
    blocks = torch.arange(row_from, row_to) // BLOCK_SIZE
    keep = (cols[None, :] >= start[blocks][:, None]) & (cols[None, :] < end[blocks][:, None])
    return torch.where(keep, k, torch.zeros((), dtype=k.dtype)) @ rhs


def time_masked_matmul(kernel_type, x1, x2, rhs, params, start, end, budget_seconds: float,
                       blocks_per_slab: int = 8):
    """Time slabs of batch item 0 until ``budget_seconds`` is used (at least one slab).

    Returns (seconds, in_band_pairs, dense_pairs, slabs, result_rows) for the rows computed.
    """
    m, n = x1.shape[0], x2.shape[0]
    row_blocks = -(-m // BLOCK_SIZE)
    done = 0
    in_band = 0
    outputs = []
    begin = time.perf_counter()
    while done < row_blocks:
        upto = min(done + blocks_per_slab, row_blocks)
        outputs.append(masked_matmul_slab(kernel_type, x1, x2, rhs, params, start, end, done, upto))
        for i in range(done, upto):
            rows = min(BLOCK_SIZE, m - i * BLOCK_SIZE)
            in_band += rows * max(int(end[i]) - int(start[i]), 0)
        done = upto
        if time.perf_counter() - begin >= budget_seconds:
            break
    seconds = time.perf_counter() - begin
    rows_done = min(done * BLOCK_SIZE, m)
    return seconds, in_band, rows_done * n, done // blocks_per_slab + (done % blocks_per_slab > 0), torch.cat(outputs)
