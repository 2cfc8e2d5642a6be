"""Pins the float64 oracle (oracle/kernels.py) against facts that do not come from it:
closed-form special cases, scipy's distance routine, GPyTorch's parametrisations written out
by hand (as the reference's tests map them, tests/conftest.py:179-226), torch.autograd and
central finite differences for the derivatives, and structural identities of the operators."""
import math

import numpy as np
import pytest
import torch
from scipy.spatial.distance import cdist

from oracle import kernels as oracle

KERNELS = ["rbf", "spectral", "locally_periodic"]


def _params(kernel_type, rng, batch=()):
    p = {"rbf": 2, "spectral": 3, "locally_periodic": 4}[kernel_type]
    return (0.5 + rng.random((*batch, p))).astype(np.float32)


def _torch_kernel(kernel_type, x1, x2, params):
    """Independent float64 torch statement of the kernels in GPyTorch's own parametrisation."""
    d = x1[..., :, None] - x2[..., None, :]
    if kernel_type == "rbf":  # ScaleKernel(RBFKernel)
        l, s = params[..., 0, None, None], params[..., 1, None, None]
        return s * torch.exp(-0.5 * (d / l) ** 2)
    if kernel_type == "spectral":  # SpectralMixtureKernel(num_mixtures=1)
        l, f, s = (params[..., i, None, None] for i in range(3))
        mixture_scale = torch.sqrt(1 / (4 * math.pi**2 * l**2))  # tests/conftest.py:196
        return s * torch.exp(-2 * math.pi**2 * d**2 * mixture_scale**2) * torch.cos(2 * math.pi * f * d)
    # ScaleKernel(RBFKernel * PeriodicKernel)
    l, lp, period, s = (params[..., i, None, None] for i in range(4))
    return s * torch.exp(-0.5 * (d / l) ** 2) * torch.exp(-2 * torch.sin(math.pi * d.abs() / period) ** 2 / lp)


@pytest.mark.parametrize("kernel_type", KERNELS)
def test_value_at_zero_distance_is_outputscale(kernel_type):
    rng = np.random.default_rng(0)
    params = _params(kernel_type, rng, (3,))
    x = rng.random((3, 5)).astype(np.float32)
    k = oracle.kernel_matrix(kernel_type, x, x, params)
    for b in range(3):
        np.testing.assert_allclose(np.diag(k[b]), params[b, -1].astype(np.float64), rtol=1e-15)
    assert np.allclose(k, np.swapaxes(k, -1, -2))  # stationary kernels are symmetric


def test_spectral_with_zero_frequency_is_rbf():
    rng = np.random.default_rng(1)
    x1, x2 = rng.random(7).astype(np.float32) * 5, rng.random(9).astype(np.float32) * 5
    k_s = oracle.kernel_matrix("spectral", x1, x2, np.array([1.3, 0.0, 0.7], dtype=np.float32))
    k_r = oracle.kernel_matrix("rbf", x1, x2, np.array([1.3, 0.7], dtype=np.float32))
    np.testing.assert_allclose(k_s, k_r, rtol=1e-15)


def test_rbf_against_scipy_cdist():
    rng = np.random.default_rng(2)
    x1, x2 = rng.random(11) * 10, rng.random(13) * 10
    l, s = 1.7, 0.6
    expected = s * np.exp(-cdist(x1[:, None], x2[:, None], "sqeuclidean") / (2 * l * l))
    got = oracle.kernel_matrix("rbf", x1, x2, np.array([l, s]))
    np.testing.assert_allclose(got, expected, rtol=1e-13)


def test_known_values():
    # hand-computed entries
    k = oracle.kernel_matrix("spectral", [1.0], [0.0], np.array([1.0, 0.25, 2.0]))
    assert abs(k[0, 0] - 2.0 * math.exp(-0.5) * math.cos(math.pi / 2)) < 1e-15
    k = oracle.kernel_matrix("spectral", [1.0], [0.0], np.array([2.0, 0.5, 3.0]))
    assert abs(k[0, 0] - 3.0 * math.exp(-0.125) * -1.0) < 1e-15
    k = oracle.kernel_matrix("locally_periodic", [0.5], [0.0], np.array([1.0, 2.0, 1.0, 1.5]))
    assert abs(k[0, 0] - 1.5 * math.exp(-0.125 - 1.0)) < 1e-15  # sin^2(pi/2) = 1, 2/lp = 1


@pytest.mark.parametrize("kernel_type", KERNELS)
def test_values_against_gpytorch_parametrisation(kernel_type):
    rng = np.random.default_rng(3)
    params = _params(kernel_type, rng, (2,))
    x1, x2 = rng.random((2, 6)).astype(np.float32) * 8, rng.random((2, 9)).astype(np.float32) * 8
    expected = _torch_kernel(kernel_type, torch.from_numpy(x1).double(), torch.from_numpy(x2).double(),
                             torch.from_numpy(params).double()).numpy()
    np.testing.assert_allclose(oracle.kernel_matrix(kernel_type, x1, x2, params), expected, rtol=1e-12, atol=1e-15)


@pytest.mark.parametrize("kernel_type", KERNELS)
def test_gradients_against_autograd_and_finite_differences(kernel_type):
    rng = np.random.default_rng(4)
    params = _params(kernel_type, rng, (2,))
    x1, x2 = rng.random((2, 5)).astype(np.float32) * 6, rng.random((2, 7)).astype(np.float32) * 6
    grad = oracle.kernel_matrix_grad(kernel_type, x1, x2, params)
    assert grad.shape == (2, params.shape[-1], 5, 7)

    pt = torch.from_numpy(params).double().requires_grad_(True)
    kt = _torch_kernel(kernel_type, torch.from_numpy(x1).double(), torch.from_numpy(x2).double(), pt)
    for i in range(5):
        for j in range(7):
            for b in range(2):
                (g,) = torch.autograd.grad(kt[b, i, j], pt, retain_graph=True)
                np.testing.assert_allclose(grad[b, :, i, j], g[b].numpy(), rtol=1e-10, atol=1e-14)

    h = 1e-6
    p64 = params.astype(np.float64)
    for p in range(params.shape[-1]):
        up, dn = p64.copy(), p64.copy()
        up[:, p] += h
        dn[:, p] -= h
        fd = (oracle.kernel_matrix(kernel_type, x1, x2, up) - oracle.kernel_matrix(kernel_type, x1, x2, dn)) / (2 * h)
        np.testing.assert_allclose(grad[:, p], fd, rtol=1e-6, atol=1e-8)


def test_range_mask_follows_block_rows():
    # rows [128 i, 128 (i+1)) x columns [start_i, end_i)  (tests/conftest.py:243-249)
    start = np.array([0, 100, 300])
    end = np.array([150, 280, 300])
    mask = oracle.range_mask(start, end, 300, 400)
    expected = np.zeros((300, 400), dtype=bool)
    expected[0:128, 0:150] = True
    expected[128:256, 100:280] = True
    assert np.array_equal(mask, expected)  # third block is empty
    small = oracle.range_mask(np.array([1, 0]), np.array([3, 2]), 5, 4, block_size=3)
    assert small.astype(int).tolist() == [[0, 1, 1, 0]] * 3 + [[1, 1, 0, 0]] * 2


@pytest.mark.parametrize("kernel_type", KERNELS)
def test_operator_identities(kernel_type):
    rng = np.random.default_rng(5)
    m, n, k = 300, 260, 3
    params = _params(kernel_type, rng, (2,))
    x1 = np.sort(rng.random((2, m)).astype(np.float32) * 10, axis=-1)
    x2 = np.sort(rng.random((2, n)).astype(np.float32) * 10, axis=-1)
    rhs = rng.standard_normal((2, n, k)).astype(np.float32)
    g = rng.standard_normal((2, m, k)).astype(np.float32)
    start = np.array([[0, 60, 150], [10, 70, 200]])
    end = np.array([[120, 200, 260], [100, 260, 260]])

    out = oracle.matmul(kernel_type, x1, x2, rhs, params, start, end)
    dense = oracle.dense(kernel_type, x1, x2, params, start, end)
    # brute force on a few entries
    for b, i, c in [(0, 0, 0), (1, 130, 2), (0, 299, 1)]:
        blk = i // 128
        acc = 0.0
        for j in range(start[b, blk], end[b, blk]):
            acc += oracle.kernel_matrix(kernel_type, x1[b, i:i + 1], x2[b, j:j + 1], params[b])[0, 0] * float(rhs[b, j, c])
        assert abs(acc - out[b, i, c]) < 1e-12
    # linear in rhs and in the outputscale
    np.testing.assert_allclose(oracle.matmul(kernel_type, x1, x2, 2 * rhs, params, start, end), 2 * out, rtol=1e-14)
    scaled = params.copy()
    scaled[:, -1] *= 3
    np.testing.assert_allclose(oracle.matmul(kernel_type, x1, x2, rhs, scaled, start, end), 3 * out, rtol=1e-6)
    # no cutoff == dense K @ rhs
    full_s, full_e = np.zeros((2, 3), dtype=int), np.full((2, 3), n)
    np.testing.assert_allclose(oracle.matmul(kernel_type, x1, x2, rhs, params, full_s, full_e),
                               oracle.kernel_matrix(kernel_type, x1, x2, params) @ rhs.astype(np.float64), rtol=1e-13)

    # parameter gradient of sum(G * (K rhs)) == autograd through the masked dense matrix
    pg = oracle.param_grad(kernel_type, x1, x2, g, rhs, params, start, end)
    pt = torch.from_numpy(params).double().requires_grad_(True)
    kt = _torch_kernel(kernel_type, torch.from_numpy(x1).double(), torch.from_numpy(x2).double(), pt)
    kt = kt * torch.from_numpy(oracle.range_mask(start, end, m, n))
    ((kt @ torch.from_numpy(rhs).double()) * torch.from_numpy(g).double()).sum().backward()
    np.testing.assert_allclose(pg, pt.grad.numpy(), rtol=1e-9, atol=1e-12)
    # d/d outputscale is the forward result contracted with G, divided by the outputscale
    np.testing.assert_allclose(pg[:, -1], (g * out).sum(axis=(-2, -1)) / params[:, -1], rtol=1e-9)

    # index: gather from the masked matrix, zero outside the pattern
    rows = rng.integers(0, m, 50)
    cols = rng.integers(0, n, 50)
    bi = rng.integers(0, 2, 50)
    got = oracle.index(kernel_type, x1, x2, params, start, end, [bi], rows, cols)
    np.testing.assert_array_equal(got, dense[bi, rows, cols])
    outside = ~oracle.range_mask(start, end, m, n)[bi, rows, cols]
    assert outside.any() and np.all(got[outside] == 0.0)


def test_count_pairs():
    assert oracle.count_pairs(np.array([0, 10]), np.array([100, 50]), 200) == 128 * 100 + 72 * 40


@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
def test_dense_cpu_baseline_matches_the_float64_oracle(kernel_type):
    """The fp32 build-K-then-matmul port that bench.py times as the CPU baseline computes the
    same masked product as the float64 closed forms (fp32 rounding apart), slab by slab."""
    import torch

    from oracle import dense_cpu
    from oracle import ranges as oracle_ranges

    g = torch.Generator().manual_seed(17)
    n, k = 1500, 7
    x = torch.sort(torch.rand(n, generator=g) * 40.0)[0]
    params = {"rbf": [1.3, 0.7], "spectral": [1.3, 0.4, 0.7],
              "locally_periodic": [1.3, 1.1, 1.7, 0.7]}[kernel_type]
    params = torch.tensor(params)
    rhs = torch.randn(n, k, generator=g)
    start, end = oracle_ranges.make_ranges(4.0, x.numpy())
    expected = oracle.matmul(kernel_type, x.numpy(), x.numpy(), rhs.numpy(), params.numpy(), start, end)
    st, en = torch.from_numpy(start), torch.from_numpy(end)
    rows = -(-n // 128)
    got = torch.cat([dense_cpu.masked_matmul_slab(kernel_type, x, x, rhs, params, st, en, b, min(b + 5, rows))
                     for b in range(0, rows, 5)])
    assert got.shape == (n, k)
    scale = np.abs(oracle.dense(kernel_type, x.numpy(), x.numpy(), params.numpy(), start, end)) @ np.abs(rhs.double().numpy())
    assert np.all(np.abs(got.double().numpy() - expected) <= 1e-5 * scale + 1e-6)
    sec, in_band, dense_pairs, slabs, out = dense_cpu.time_masked_matmul(
        kernel_type, x, x, rhs, params, st, en, budget_seconds=0.0, blocks_per_slab=4)
    assert slabs == 1 and out.shape == (512, k) and dense_pairs == 512 * n
    assert in_band == oracle.count_pairs(start[:4], end[:4], 512)
    assert torch.equal(out, got[:512]) or torch.allclose(out, got[:512], rtol=0, atol=1e-5)
