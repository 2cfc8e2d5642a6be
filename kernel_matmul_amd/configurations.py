"""Configuration objects: operator arguments -> define dict(s) and cache keys.

Class names, constructor signatures and the keys of the returned dicts are those of the
reference (kernel_matmul/configurations.py:11-254) because callers and tests construct them
directly and edit the dicts.  The reference's autotune search space (3 thread shapes x 4
column splits x K-block sizes, :94-118) is replaced by a small gfx950 table: the device code
is compiled ahead of time and the only degrees of freedom left are the number of wavefronts
sharing a row range and the rows per wavefront, which the library's launch table already
picks from the problem size.
"""
from __future__ import annotations

import abc
import math
from typing import Any

from torch import Tensor

from kernel_matmul_amd import _BLOCK_SIZE
from kernel_matmul_amd.compile import Defines

_KERNEL_DEFINE = {
    "rbf": "KERNEL_RBF",
    "spectral": "KERNEL_SPECTRAL",
    "locally_periodic": "KERNEL_LOCALLY_PERIODIC",
    "compact": "KERNEL_COMPACT",
}


def get_kernel_type_defines(kernel_type: str, params: Tensor) -> dict[str, Any]:
    defines: dict[str, Any] = {_KERNEL_DEFINE[kernel_type]: None}
    if kernel_type == "compact":
        defines["NUM_ORDERS"] = int(math.sqrt(params.shape[-1] - 0.75))
    return defines


def augment_cache_key(key: str, kernel_type: str, params: Tensor) -> str:
    return f"{key}_{params.shape[-1]}" if kernel_type == "compact" else key


class Configuration(abc.ABC):
    """Maps operator arguments to candidate define sets and to a cache key."""

    @abc.abstractmethod
    def make_candidates(self, args: tuple) -> list[Defines]:
        ...

    @abc.abstractmethod
    def cache_key(self, args: tuple) -> str:
        ...


class SingleConfiguration(Configuration):
    """A configuration with exactly one candidate."""

    def make_candidates(self, args: tuple) -> list[Defines]:
        return [self.make_config(args)]

    @abc.abstractmethod
    def make_config(self, args: tuple) -> Defines:
        ...


class _KernelTypeConfiguration(SingleConfiguration):
    """Shared plumbing: every operator's defines start with block size, batch rank, kernel."""

    #: position of ``params`` in the operator's argument tuple
    params_position = 3
    #: operator-specific defines
    extra: dict[str, Any] = {}

    def __init__(self, kernel_type: str):
        self.kernel_type = kernel_type

    def _base(self, args: tuple) -> Defines:
        x1 = args[0]
        return {"BLOCK_SIZE": _BLOCK_SIZE, "BATCH_DIM": x1.dim() - 1}

    def _key_parts(self, args: tuple) -> list[Any]:
        return [args[0].dim() - 1]

    def make_config(self, args: tuple) -> Defines:
        params = args[self.params_position]
        return {**self._base(args), **self.extra, **self._extra_for(args),
                **get_kernel_type_defines(self.kernel_type, params)}

    def _extra_for(self, args: tuple) -> dict[str, Any]:
        return {}

    def cache_key(self, args: tuple) -> str:
        key = "_".join(str(part) for part in self._key_parts(args))
        return augment_cache_key(key, self.kernel_type, args[self.params_position])


def _matmul_tile_defaults(k: int) -> dict[str, Any]:
    # Legacy keys kept so that callers which edit them keep working; on gfx950 only
    # MATMUL_COL_BLOCKS influences the launch.
    return {
        "MATMUL_K_BLOCK_SIZE": min(k, 32),
        "MATMUL_THREADS": 64,
        "MATMUL_PER_THREAD": 2,
        "MATMUL_COL_BLOCKS": 1,
        "MATMUL_USE_SHM": 1,
    }


class MatmulSingleConfiguration(_KernelTypeConfiguration):
    def _extra_for(self, args: tuple) -> dict[str, Any]:
        return _matmul_tile_defaults(args[2].shape[-1])

    def _key_parts(self, args: tuple) -> list[Any]:
        return [args[0].dim() - 1, args[2].shape[-1]]


class MatmulAutotuneConfiguration(Configuration):
    """gfx950 table in place of the reference's 12-36 candidate search.

    Exactly one candidate is returned: the library's own launch table (rows per wavefront,
    wavefronts per row range) is keyed on row blocks x batch items x rhs column groups and has
    been tuned offline, so there is nothing left to time at run time.
    """

    def __init__(self, kernel_type: str):
        self.kernel_type = kernel_type

    def make_candidates(self, args: tuple) -> list[Defines]:
        x1, x2, rhs, params, start, end = args
        candidate = {
            "BLOCK_SIZE": _BLOCK_SIZE,
            "BATCH_DIM": x1.dim() - 1,
            **_matmul_tile_defaults(rhs.shape[-1]),
            **get_kernel_type_defines(self.kernel_type, params),
        }
        if self.kernel_type == "compact":
            candidate["KERNEL_COMPACT_NUM_ORDERS"] = int(math.sqrt(params.shape[-1] - 0.75))
        return [candidate]

    def cache_key(self, args: tuple) -> str:
        x1, x2, rhs, params, start, end = args
        return augment_cache_key(f"{x1.dim() - 1}_{rhs.shape[-1]}", self.kernel_type, params)


class MatmulBwdConfiguration(_KernelTypeConfiguration):
    extra = {"MATMUL_BWD_THREAD_DIM": 16, "MATMUL_BWD_PER_THREAD": 8}


class BilinearDerivativeConfiguration(_KernelTypeConfiguration):
    params_position = 4
    extra = {"BILINEAR_DERIVATIVE_THREAD_DIM": 16, "BILINEAR_DERIVATIVE_PER_THREAD": 8}


class IndexConfiguration(_KernelTypeConfiguration):
    params_position = 2

    def _extra_for(self, args: tuple) -> dict[str, Any]:
        return {"INDEX_THREAD_DIM": 64, "INDEX_BATCH_DIM": args[6].dim() - 1}

    def _key_parts(self, args: tuple) -> list[Any]:
        return [args[0].dim() - 1, args[6].dim() - 1]


class IndexBwdConfiguration(_KernelTypeConfiguration):
    params_position = 2

    def _extra_for(self, args: tuple) -> dict[str, Any]:
        return {"INDEX_BWD_THREAD_DIM": 64, "INDEX_BWD_BATCH_DIM": args[6].dim() - 1}

    def _key_parts(self, args: tuple) -> list[Any]:
        return [args[0].dim() - 1, args[6].dim() - 1]


class DenseConfiguration(_KernelTypeConfiguration):
    params_position = 2
    extra = {"DENSE_THREAD_DIM": 16}


class DenseBwdConfiguration(_KernelTypeConfiguration):
    params_position = 2
    extra = {"DENSE_BWD_THREAD_DIM": 16}
