"""The C-ABI library loads, exports every function include/kernel_matmul_amd.h declares, and
its argument validation works without touching a GPU (no compute calls here)."""
import ctypes
import os
import re

import numpy as np
import pytest

from kernel_matmul_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "kernel_matmul_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(km_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for required in ("km_matmul", "km_param_grad", "km_param_grad_workspace_size", "km_param_grad_static", "km_index",
                     "km_make_ranges", "km_make_ranges_symmetric", "km_transpose_ranges",
                     "km_make_ranges_device", "km_make_ranges_symmetric_device", "km_last_error",
                     "km_version", "km_num_params"):
        assert required in names


def test_library_exports_every_declared_symbol():
    lib = _native.load_library()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_version_and_num_params():
    lib = _native.load_library()
    assert lib.km_version() >= 100
    assert [lib.km_num_params(i) for i in range(4)] == [2, 3, 4, -1]


def test_host_argument_validation():
    lib = _native.load_library()
    x = np.zeros(4, dtype=np.float32)
    out = np.zeros(4, dtype=np.int32)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    status = lib.km_make_ranges_symmetric(p(x), 1, 4, 1.0, 0, p(out), p(out))
    assert status == -1 and b"block_size" in lib.km_last_error()
    status = lib.km_make_ranges(None, None, 1, 4, 4, 1.0, 2, 0, p(out), p(out))
    assert status == -1 and b"NULL" in lib.km_last_error()
    status = lib.km_transpose_ranges(p(out), p(out), 1, 3, 4, 4, 2, p(out), p(out))
    assert status == -1 and b"rows" in lib.km_last_error()


def test_device_entry_points_reject_bad_arguments_before_launching():
    lib = _native.load_library()
    sizes = (ctypes.c_int64 * 1)(2)
    # unknown kernel type
    status = lib.km_matmul(9, 1, sizes, 4, 4, 1, None, None, None, None, None, None, None, None,
                           None, None, None, None, None, None, None)
    assert status == -2 and b"kernel type" in lib.km_last_error()
    # too many batch dimensions
    status = lib.km_matmul(0, 7, sizes, 4, 4, 1, None, None, None, None, None, None, None, None,
                           None, None, None, None, None, None, None)
    assert status == -2 and b"batch rank" in lib.km_last_error()
    # NULL data pointer
    status = lib.km_matmul(0, 1, sizes, 4, 4, 1, None, None, None, None, None, None, None, None,
                           None, None, None, None, None, None, None)
    assert status == -1 and b"NULL" in lib.km_last_error()
    # empty problems are accepted and do nothing
    assert lib.km_matmul(0, 1, sizes, 0, 4, 1, None, None, None, None, None, None, None, None,
                         None, None, None, None, None, None, None) == 0
    assert lib.km_param_grad_workspace_size(1, 1, sizes, 1000, 1000, 4) > 0
    assert lib.km_param_grad_workspace_size(1, 1, sizes, 0, 1000, 4) == 0
    # the allocation-free variant refuses problems beyond its static scratch before anything else
    many = (ctypes.c_int64 * 1)(64)
    assert lib.km_param_grad_workspace_size(0, 1, many, 1_000_000, 1_000_000, 2) > 4 << 20
    status = lib.km_param_grad_static(0, 1, many, 1_000_000, 1_000_000, 2, *([None] * 14), None, None)
    assert status == -4 and b"static buffer" in lib.km_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", "/nonexistent/libkernel_matmul_amd.so")
    with pytest.raises(RuntimeError, match="native library not found"):
        _native.load_library()


def test_launch_descriptions_without_a_gpu():
    """km_matmul_describe / km_param_grad_describe report the launch tables' choices (host only)."""
    text = _native.describe_matmul("spectral", 8, 100_000, 100_000, 16, None)
    assert "fwd_table_f16_grouped<spectral>" in text and "128 rows per wavefront" in text
    assert "fwd_table_f16<spectral, G=2" in _native.describe_matmul("spectral", 8, 1_000_000, 1_000_000, 32, None)
    assert "fwd_mfma_f16<spectral, G=4" in _native.describe_matmul("spectral", 8, 1_000_000, 1_000_000, 64, None)
    assert "fwd_mfma_f16<rbf, G=2" in _native.describe_matmul("rbf", 8, 1_000_000, 1_000_000, 32, None)
    assert "fwd_table_f16_grouped<rbf>" in _native.describe_matmul("rbf", 8, 1_000_000, 1_000_000, 16, None)
    assert "fwd_block<locally_periodic" in _native.describe_matmul("locally_periodic", 8, 1_000_000, 1_000_000, 16, None)
    # narrow vectors: feature form; wide ones and the locally periodic kernel: pairwise form
    assert "param_grad_features<spectral, GE=2" in _native.describe_param_grad("spectral", 16, 100_000, 4)
    assert "param_grad_partial<spectral, TL=2>" in _native.describe_param_grad("spectral", 2, 50_000, 8)
    assert "param_grad_features<rbf, GE=2" in _native.describe_param_grad("rbf", 2, 50_000, 10)
    assert "param_grad_partial<locally_periodic" in _native.describe_param_grad("locally_periodic", 2, 5_000, 3)
    lib = _native.load_library()
    buf = ctypes.create_string_buffer(16)
    assert lib.km_param_grad_describe(7, 1, 128, 4, buf, len(buf)) == -2
    assert lib.km_param_grad_describe(1, 1, 128, 4, None, 0) == -1
    # a failed status reaches Python as RuntimeError with the library's message
    with pytest.raises(RuntimeError, match="km_param_grad_describe: invalid argument"):
        _native.describe_param_grad("spectral", 1, -5, 4)
    with pytest.raises(RuntimeError, match="km_matmul_describe: invalid argument"):
        _native.describe_matmul("spectral", 1, -5, 10, 4)
