"""Loader of the native operators and the timing helpers.

The reference JIT-compiles one CUDA module per (operator, define set) and autotunes over
define sets (kernel_matmul/compile.py:49-125, 148-201).  Here every operator is compiled
ahead of time into one gfx950 library; ``load_native(name, defines)`` keeps its signature and
returns an object with ``.call(*args)``, and the define dict only selects the kernel function
and, for ``matmul``, nudges the launch table.
"""
from __future__ import annotations

import multiprocessing
import multiprocessing.pool
import os
from contextlib import contextmanager
from typing import Any, Callable

import torch

from kernel_matmul_amd import _BLOCK_SIZE, _native

Defines = dict[str, Any]

_global_compile_pool: multiprocessing.pool.Pool | None = None

_KERNEL_DEFINES = {
    "KERNEL_RBF": "rbf",
    "KERNEL_SPECTRAL": "spectral",
    "KERNEL_LOCALLY_PERIODIC": "locally_periodic",
}

_OPERATORS = ("matmul", "matmul_bwd", "bilinear_derivative", "index", "index_bwd", "dense",
              "dense_bwd")


@contextmanager
def compile_pool(processes: int):
    """Process-wide worker pool, kept for source compatibility.

    Nothing is compiled at run time any more, so the pool never receives work; opening two at
    once is still an error, as in the reference (kernel_matmul/compile.py:24-46).
    """
    global _global_compile_pool
    if _global_compile_pool is not None:
        raise RuntimeError("compile_pool is already active")
    _global_compile_pool = multiprocessing.get_context("spawn").Pool(processes)
    try:
        yield
    finally:
        _global_compile_pool.close()
        _global_compile_pool.join()
        _global_compile_pool = None


def get_native_module_path(name: str) -> str:
    """Directory holding the native sources (all operators share ``csrc``)."""
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def _debug_enabled() -> bool:
    return os.environ.get("KERNEL_MATMUL_COMPILE_DEBUG", "false") == "true"


class NativeModule:
    """One operator bound to a kernel type: what ``load_native`` returns.

    ``name`` follows the reference's module naming (``km___<op>___<KEY>__<VALUE>...``,
    kernel_matmul/compile.py:90-104) so logs and caches keyed on it keep working.
    """

    def __init__(self, op: str, defines: Defines):
        if op not in _OPERATORS:
            raise ValueError(f"Unknown native module: {op}")
        kernel_types = [value for key, value in _KERNEL_DEFINES.items() if key in defines]
        if "KERNEL_COMPACT" in defines:
            raise NotImplementedError("the compact kernel is not available in this build")
        if len(kernel_types) != 1:
            raise ValueError("No kernel function defined" if not kernel_types
                             else "More than one kernel function defined")
        block = defines.get("BLOCK_SIZE", _BLOCK_SIZE)
        if block != _BLOCK_SIZE:
            raise ValueError(f"BLOCK_SIZE must be {_BLOCK_SIZE}, got {block}")
        self.op = op
        self.kernel_type = kernel_types[0]
        self.defines = dict(defines)
        self.debug = _debug_enabled()
        self.print_size = os.environ.get("KERNEL_MATMUL_COMPILE_PRINT_SIZE", "false") == "true"
        self.name = "km___" + op + "".join(
            f"___{key}" if defines[key] is None else f"___{key}__{defines[key]}"
            for key in sorted(defines)
        ) + ("___debug" if self.debug else "")
        self._options = self._launch_options()
        _native.load_library()

    def _launch_options(self):
        """Legacy tile defines -> launch table overrides (matmul only).

        ``MATMUL_COL_BLOCKS`` asked the reference kernel to split a row block's column range
        over several thread blocks (native/matmul/matmul.cu:33-34, 70-72); here it becomes the
        number of wavefronts sharing a row range.  Thread-shape defines have no equivalent.
        """
        if self.op != "matmul":
            return None
        options = _native.LaunchOptions()
        col_blocks = self.defines.get("MATMUL_COL_BLOCKS")
        if col_blocks is not None and col_blocks > 1:
            options.col_splits = min(int(col_blocks), 8)
        variant = self.defines.get("MATMUL_VARIANT")
        if variant is not None:
            options.variant = {"auto": 0, "valu": 1, "mfma": 2, "mfma_f32": 2, "mfma_f16": 3, "mfma_f16_direct": 4,
                               "block": 5, "mfma_f32_direct": 6}[variant]
        if self.defines.get("MATMUL_TAIL_BALANCE") == 0:
            options.reserved = 1
        elif self.defines.get("MATMUL_GROUP_TAIL") is not None:
            options.reserved = 2 + min(int(self.defines["MATMUL_GROUP_TAIL"]), 0xFFFF)
            halves = self.defines.get("MATMUL_GROUP_TAIL_HALVES")
            if halves is not None:
                options.reserved += (min(int(halves), 0x3FFF) + 1) << 16
        rows = self.defines.get("MATMUL_ROWS_PER_WAVE")
        if rows is not None:
            options.rows_per_wave = int(rows)
        return options

    def describe(self, *args) -> str:
        """Which kernel and decomposition ``call(*args)`` runs, as the library's launch tables
        report it for matmul and the parameter gradients (nothing is launched)."""
        if self.op in ("matmul_bwd", "bilinear_derivative"):
            x1, left = args[0], args[2]
            batches = 1
            for size in x1.shape[:-1]:
                batches *= size
            return _native.describe_param_grad(self.kernel_type, batches, x1.shape[-1], left.shape[-1])
        if self.op != "matmul":
            return {"index": "km::index_kernel", "index_bwd": "km::index_bwd_terms + reduce",
                    "dense": "km::dense_kernel", "dense_bwd": "km::dense_bwd_partial + reduce"}[self.op]
        x1, x2, rhs = args[0], args[1], args[2]
        batches = 1
        for size in x1.shape[:-1]:
            batches *= size
        return _native.describe_matmul(self.kernel_type, batches, x1.shape[-1], x2.shape[-1], rhs.shape[-1],
                                       self._options)

    def _check_batch_dim(self, x1) -> None:
        declared = self.defines.get("BATCH_DIM")
        if declared is not None and declared != x1.dim() - 1:
            raise RuntimeError(
                f"module was specialised for {declared} batch dimension(s), got {x1.dim() - 1}"
            )

    def call(self, *args):
        kt = self.kernel_type
        if self.op == "matmul":
            x1, x2, rhs, params, start, end = args
            self._check_batch_dim(x1)
            if self.print_size:
                print(f"m, n, k: ({x1.shape[-1]}, {x2.shape[-1]}, {rhs.shape[-1]})")
            result = _native.matmul(kt, x1, x2, rhs, params, start, end, self._options)
        elif self.op == "matmul_bwd":
            x1, x2, rhs, params, start, end, out_grad = args
            self._check_batch_dim(x1)
            result = _native.param_grad(kt, x1, x2, out_grad, rhs, params, start, end)
        elif self.op == "bilinear_derivative":
            x1, x2, left_vecs, right_vecs, params, start, end = args
            self._check_batch_dim(x1)
            result = _native.param_grad(kt, x1, x2, left_vecs, right_vecs, params, start, end)
        elif self.op == "index":
            x1, x2, params, start, end, batch_indices, row_index, col_index = args
            self._check_batch_dim(x1)
            result = _native.index(kt, x1, x2, params, start, end, batch_indices, row_index,
                                   col_index)
        elif self.op == "index_bwd":
            x1, x2, params, start, end, batch_indices, row_index, col_index, out_grad = args
            self._check_batch_dim(x1)
            result = _native.index_bwd(kt, x1, x2, params, start, end, batch_indices, row_index,
                                       col_index, out_grad)
        elif self.op == "dense":
            x1, x2, params, start, end = args
            self._check_batch_dim(x1)
            result = _native.dense(kt, x1, x2, params, start, end)
        else:
            x1, x2, params, start, end, out_grad = args
            self._check_batch_dim(x1)
            result = _native.dense_bwd(kt, x1, x2, params, start, end, out_grad)
        if self.debug:
            # Debug builds of the reference synchronise and check after every launch
            # (native/common/gpu_assert.cuh:6-23).
            torch.cuda.synchronize(result.device)
        return result


def load_native(name: str, defines: Defines | None = None) -> NativeModule:
    """Return the operator ``name`` specialised by ``defines`` (an object with ``.call``)."""
    return NativeModule(name, {} if defines is None else defines)


def find_best(
    name: str,
    args: list[Any],
    candidates: list[Defines],
    return_timings: bool = False,
    num_measurements: int = 1,
    compile_pool: multiprocessing.pool.Pool | None = None,
) -> dict[str, Any] | tuple[dict[str, Any], list[float]]:
    """Time every candidate on ``args`` and return the fastest (optionally with all timings)."""
    timings = []
    for candidate in candidates:
        module = load_native(name, defines=candidate)
        samples = cuda_time(lambda: module.call(*args), num_measurements=num_measurements)
        timings.append(sum(samples) / len(samples))
    best = candidates[min(range(len(candidates)), key=timings.__getitem__)]
    return (best, timings) if return_timings else best


def cuda_time(fn: Callable, num_measurements: int | None = None) -> float | list[float]:
    """Milliseconds per call of ``fn`` measured with events on the current stream."""
    count = 1 if num_measurements is None else num_measurements
    timings = []
    for _ in range(count):
        begin = torch.cuda.Event(enable_timing=True)
        finish = torch.cuda.Event(enable_timing=True)
        begin.record()
        fn()
        finish.record()
        finish.synchronize()
        timings.append(begin.elapsed_time(finish))
    return timings[0] if num_measurements is None else timings
