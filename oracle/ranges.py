"""ctypes front end of the C range-builder oracle (ranges_oracle.c).  TEST INFRASTRUCTURE.

Mirrors the batch handling of the reference's Python wrapper (kernel_matmul/ranges.py:39-127):
batch dimensions are flattened to one, ``cutoff=None`` yields the dense pattern, ``x2=None``
selects the symmetric builder, and an unaligned pattern cannot be transposed.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkm_ranges_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s", "libkm_ranges_oracle.so"], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int32)
        _lib.oracle_make_ranges.argtypes = [fp, fp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_float, ctypes.c_int, ctypes.c_int, ip, ip]
        _lib.oracle_make_ranges.restype = None
        _lib.oracle_make_ranges_symmetric.argtypes = [fp, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                      ctypes.c_int, ip, ip]
        _lib.oracle_make_ranges_symmetric.restype = None
        _lib.oracle_transpose_ranges.argtypes = [ip, ip, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_int, ctypes.c_int, ip, ip]
        _lib.oracle_transpose_ranges.restype = None
    return _lib


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _iptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


def make_ranges(cutoff, x1, x2=None, *, block_size: int = 128, align: bool = False):
    lib = _load()
    x1 = np.ascontiguousarray(x1, dtype=np.float32)
    batch_shape = x1.shape[:-1]
    n1 = x1.shape[-1]
    x1f = x1.reshape(-1, n1)
    nb = x1f.shape[0]
    rows = int(math.ceil(n1 / block_size))
    if x2 is not None:
        x2 = np.ascontiguousarray(x2, dtype=np.float32)
        n2 = x2.shape[-1]
        x2f = x2.reshape(-1, n2)
    else:
        n2 = n1
    start = np.zeros((nb, rows), dtype=np.int32)
    end = np.zeros((nb, rows), dtype=np.int32)
    if cutoff is None:
        end[:] = n2
    elif x2 is None:
        lib.oracle_make_ranges_symmetric(_fptr(x1f), nb, n1, float(cutoff), block_size,
                                         _iptr(start), _iptr(end))
    else:
        lib.oracle_make_ranges(_fptr(x1f), _fptr(x2f), nb, n1, n2, float(cutoff), block_size,
                               int(bool(align)), _iptr(start), _iptr(end))
    return start.reshape(*batch_shape, rows), end.reshape(*batch_shape, rows)


def transpose_ranges(start, end, x1_size: int, x2_size: int, *, block_size: int = 128):
    lib = _load()
    start = np.ascontiguousarray(start, dtype=np.int32)
    end = np.ascontiguousarray(end, dtype=np.int32)
    if np.any((start % block_size != 0) & (start != x2_size)) or np.any(
        (end % block_size != 0) & (end != x2_size)
    ):
        raise ValueError("Ranges must be block-aligned")
    batch_shape = start.shape[:-1]
    rows = start.shape[-1]
    sf = start.reshape(-1, rows)
    ef = end.reshape(-1, rows)
    nb = sf.shape[0]
    cols = int(math.ceil(x2_size / block_size))
    start_t = np.zeros((nb, cols), dtype=np.int32)
    end_t = np.zeros((nb, cols), dtype=np.int32)
    lib.oracle_transpose_ranges(_iptr(sf), _iptr(ef), nb, rows, x1_size, x2_size, block_size,
                                _iptr(start_t), _iptr(end_t))
    return start_t.reshape(*batch_shape, cols), end_t.reshape(*batch_shape, cols)
