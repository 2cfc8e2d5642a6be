"""Callable wrapper around a native operator (reference: kernel_matmul/native_function.py:11-86).

``NativeFunction(name, config)(*args)`` asks the configuration for a cache key; when the key
changes (different batch rank, rhs width, ...) it asks for candidate define sets, times them if
there is more than one, and binds the winner through ``load_native``.  With the gfx950 table
the configurations return one candidate, so the timing branch only runs for caller-supplied
configurations with several.
"""
from __future__ import annotations

import multiprocessing.pool
from typing import Any

from kernel_matmul_amd.compile import Defines, find_best, load_native
from kernel_matmul_amd.configurations import Configuration
from kernel_matmul_amd.util import format_dict


class NativeFunction:
    def __init__(
        self,
        name: str,
        config: Configuration,
        num_measurements: int = 1,
        verbose: bool = False,
        compile_pool: multiprocessing.pool.Pool | None = None,
    ):
        self.name = name
        self.config = config
        self.num_measurements = num_measurements
        self.verbose = verbose
        self.compile_pool = compile_pool
        self._defines: Defines | None = None
        self._cache_key: str | None = None
        self._module = None

    def _select(self, args: tuple) -> Defines:
        candidates = self.config.make_candidates(args)
        if len(candidates) == 1:
            return candidates[0]
        if self.verbose:
            print(f"Autotuning {self.name}...")
        best, timings = find_best(
            self.name,
            args,
            candidates,
            return_timings=True,
            num_measurements=self.num_measurements,
            compile_pool=self.compile_pool,
        )
        if self.verbose:
            for position, (timing, candidate) in enumerate(zip(timings, candidates)):
                print(f"  - Candidate {position}: {timing:.3f} ms ({format_dict(candidate)})")
            print(f"Best: {format_dict(best)}")
        return best

    def __call__(self, *args: Any) -> Any:
        key = self.config.cache_key(args)
        if self._module is None or key != self._cache_key:
            self._defines = self._select(args)
            self._module = load_native(self.name, defines=self._defines)
            self._cache_key = key
        return self._module.call(*args)

    @property
    def defines(self) -> Defines | None:
        """Define set bound by the last (re)selection; ``None`` before the first call."""
        return self._defines
