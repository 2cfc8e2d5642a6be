"""Float64 closed-form oracle of the kernel functions and the operators built on them.

TEST INFRASTRUCTURE: imported by tests, smoke() and bench.py's cpu_baseline only.

What each function restates (reference = Turakar/kernel-matmul):

* ``kernel_matrix``      native/common/kernel_function.cuh:25-58 composed with the parameter
                         transform at :198-219, i.e. in terms of the *user* parameters
                         rbf [l, s]:                s exp(-d^2 / (2 l^2))
                         spectral [l, f, s]:        s exp(-d^2 / (2 l^2)) cos(2 pi f d)
                         locally_periodic [l, lp, T, s]:
                                                    s exp(-d^2 / (2 l^2) - (2/lp) sin^2(pi d / T))
                         These are the textbook RBF, one-component spectral-mixture and
                         RBF x periodic kernels the reference's tests map to GPyTorch
                         (tests/conftest.py:179-226).
* ``kernel_matrix_grad`` native/common/kernel_function.cuh:92-163 composed with the chain rule
                         at :221-251 (derivatives w.r.t. the user parameters).
* ``range_mask``         tests/conftest.py:243-249 (rows of block i x columns [start_i, end_i)).
* ``matmul``             native/matmul/matmul.cu:160-203 == masked K @ rhs
                         (tests/native/test_matmul.py:28).
* ``param_grad``         native/matmul_bwd/matmul_bwd.cu:203-220 and
                         native/bilinear_derivative/bilinear_derivative.cu:152-182: gradient of
                         sum((left @ right^T) * masked K) w.r.t. the user parameters.
* ``index``              native/index/index.cu:36-56.
* ``dense``              native/dense/dense.cu:12-71 (masked K itself).

Pinning (tests/test_oracle_kernels.py): values at d = 0, the f = 0 reduction of spectral to
rbf, agreement with scipy's squared-euclidean cdist form, GPyTorch's spectral-mixture
parametrisation written out by hand, derivatives against torch.autograd in float64 and
central finite differences, and the matmul_bwd == bilinear_derivative identity.  No function
in this file is "parity unpinned".
"""
from __future__ import annotations

import numpy as np

BLOCK_SIZE = 128

NUM_PARAMS = {"rbf": 2, "spectral": 3, "locally_periodic": 4}


def _f64(a):
    return np.asarray(a, dtype=np.float64)


def _diff(x1, x2):
    x1 = _f64(x1)
    x2 = _f64(x2)
    return x1[..., :, None] - x2[..., None, :]


def _p(params, i):
    return _f64(params)[..., i, None, None]


def kernel_matrix(kernel_type: str, x1, x2, params) -> np.ndarray:
    """Dense K[..., m, n] in float64 from fp32-valued inputs."""
    d = _diff(x1, x2)
    if kernel_type == "rbf":
        l, s = _p(params, 0), _p(params, 1)
        return s * np.exp(-(d * d) / (2.0 * l * l))
    if kernel_type == "spectral":
        l, f, s = _p(params, 0), _p(params, 1), _p(params, 2)
        return s * np.exp(-(d * d) / (2.0 * l * l)) * np.cos(2.0 * np.pi * f * d)
    if kernel_type == "locally_periodic":
        l, lp, T, s = _p(params, 0), _p(params, 1), _p(params, 2), _p(params, 3)
        sn = np.sin(np.pi * d / T)
        return s * np.exp(-(d * d) / (2.0 * l * l) - (2.0 / lp) * sn * sn)
    raise ValueError(f"Unknown kernel type: {kernel_type}")


def kernel_matrix_grad(kernel_type: str, x1, x2, params) -> np.ndarray:
    """dK/dparams[..., P, m, n] in float64 (user parameters)."""
    d = _diff(x1, x2)
    k = kernel_matrix(kernel_type, x1, x2, params)
    if kernel_type == "rbf":
        l, s = _p(params, 0), _p(params, 1)
        return np.stack([k * d * d / l**3, k / s], axis=-3)
    if kernel_type == "spectral":
        l, f, s = _p(params, 0), _p(params, 1), _p(params, 2)
        e = np.exp(-(d * d) / (2.0 * l * l))
        g_l = k * d * d / l**3
        g_f = -2.0 * np.pi * d * s * e * np.sin(2.0 * np.pi * f * d)
        g_s = e * np.cos(2.0 * np.pi * f * d)
        return np.stack([g_l, g_f, g_s], axis=-3)
    if kernel_type == "locally_periodic":
        l, lp, T, s = _p(params, 0), _p(params, 1), _p(params, 2), _p(params, 3)
        a = np.pi * d / T
        sn, cs = np.sin(a), np.cos(a)
        g_l = k * d * d / l**3
        g_lp = k * 2.0 * sn * sn / lp**2
        g_T = k * (2.0 / lp) * 2.0 * sn * cs * np.pi * d / T**2
        g_s = k / s
        return np.stack([g_l, g_lp, g_T, g_s], axis=-3)
    raise ValueError(f"Unknown kernel type: {kernel_type}")


def range_mask(start, end, m: int, n: int, block_size: int = BLOCK_SIZE) -> np.ndarray:
    """mask[..., i, j] = start[..., i // bs] <= j < end[..., i // bs]."""
    start = np.asarray(start, dtype=np.int64)
    end = np.asarray(end, dtype=np.int64)
    block = np.arange(m) // block_size
    cols = np.arange(n)
    s = start[..., block][..., :, None]
    e = end[..., block][..., :, None]
    return (cols >= s) & (cols < e)


def dense(kernel_type, x1, x2, params, start, end, block_size: int = BLOCK_SIZE) -> np.ndarray:
    k = kernel_matrix(kernel_type, x1, x2, params)
    mask = range_mask(start, end, k.shape[-2], k.shape[-1], block_size)
    return np.where(mask, k, 0.0)


def matmul(kernel_type, x1, x2, rhs, params, start, end, block_size: int = BLOCK_SIZE) -> np.ndarray:
    return dense(kernel_type, x1, x2, params, start, end, block_size) @ _f64(rhs)


def param_grad(kernel_type, x1, x2, left, right, params, start, end,
               block_size: int = BLOCK_SIZE) -> np.ndarray:
    """grad[..., P] of sum((left @ right^T) * masked K) w.r.t. the user parameters."""
    g = kernel_matrix_grad(kernel_type, x1, x2, params)
    mask = range_mask(start, end, g.shape[-2], g.shape[-1], block_size)
    coeff = _f64(left) @ np.swapaxes(_f64(right), -1, -2)
    return np.sum(np.where(mask, coeff, 0.0)[..., None, :, :] * g, axis=(-2, -1))


def index(kernel_type, x1, x2, params, start, end, batch_indices, row_index, col_index,
          block_size: int = BLOCK_SIZE) -> np.ndarray:
    k = dense(kernel_type, x1, x2, params, start, end, block_size)
    idx = tuple(np.asarray(b, dtype=np.int64) for b in batch_indices)
    return k[idx + (np.asarray(row_index, dtype=np.int64), np.asarray(col_index, dtype=np.int64))]


def count_pairs(start, end, m: int, block_size: int = BLOCK_SIZE) -> int:
    """Number of evaluated (row, col) pairs: sum_i rows_in_block_i * (end_i - start_i)."""
    start = np.asarray(start, dtype=np.int64)
    end = np.asarray(end, dtype=np.int64)
    rows = start.shape[-1]
    rows_in_block = np.minimum(block_size, m - block_size * np.arange(rows))
    return int(np.sum(rows_in_block * np.maximum(end - start, 0)))
