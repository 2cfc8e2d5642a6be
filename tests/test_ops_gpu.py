"""GPU parity of the four device operators against the float64 oracle, through the same
``load_native(name, defines).call(*args)`` path the reference's tests use
(tests/native/test_matmul.py, test_matmul_bwd.py, test_bilinear_derivative.py, test_index.py).

Tolerances: forward/index rtol 1e-4 / atol 1e-5 (tighter than the reference's atol 2e-4);
gradients rtol 1e-4 / atol 1e-5 relative to the gradient scale (reference: 2e-3)."""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.compile import load_native
from kernel_matmul_amd.configurations import (
    BilinearDerivativeConfiguration,
    IndexConfiguration,
    MatmulBwdConfiguration,
    MatmulSingleConfiguration,
)
from oracle import kernels as oracle

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def assert_close(actual: torch.Tensor, expected: np.ndarray, rtol=RTOL, atol=ATOL):
    actual = actual.detach().cpu().double().numpy()
    assert actual.shape == expected.shape
    err = np.abs(actual - expected)
    tol = atol + rtol * np.abs(expected)
    worst = np.unravel_index(np.argmax(err - tol), err.shape) if err.size else None
    assert np.all(err <= tol), (
        f"max violation at {worst}: got {actual[worst]}, expected {expected[worst]}, "
        f"err {err[worst]:.3e} > tol {tol[worst]:.3e}"
    )


@pytest.mark.parametrize("col_blocks", [1, 2, 3, 7])
def test_matmul(example_data, col_blocks):
    d = example_data
    args = (d.x1, d.x2, d.rhs, d.params, d.start, d.end)
    defines = MatmulSingleConfiguration(d.kernel_type).make_config(args)
    assert "MATMUL_COL_BLOCKS" in defines
    defines["MATMUL_COL_BLOCKS"] = col_blocks
    result = load_native("matmul", defines).call(*args)
    a = d.numpy()
    expected = oracle.matmul(d.kernel_type, a["x1"], a["x2"], a["rhs"], a["params"], a["start"], a["end"])
    assert_close(result, expected)


@pytest.mark.parametrize("variant,rows", [("valu", None), ("mfma_f32", 16), ("mfma_f32", 32), ("mfma_f32", 64), ("mfma_f32", 128),
                                          ("mfma_f32_direct", 32), ("mfma_f32_direct", 128),
                                          ("mfma_f16", 16), ("mfma_f16", 32), ("mfma_f16", 64), ("mfma_f16", 128),
                                          ("mfma_f16_direct", 32), ("mfma_f16_direct", 128), ("block", None)])
def test_matmul_variants(example_data, variant, rows):
    d = example_data
    args = (d.x1, d.x2, d.rhs, d.params, d.start, d.end)
    defines = MatmulSingleConfiguration(d.kernel_type).make_config(args)
    defines["MATMUL_VARIANT"] = variant
    if rows is not None:
        defines["MATMUL_ROWS_PER_WAVE"] = rows
    result = load_native("matmul", defines).call(*args)
    a = d.numpy()
    expected = oracle.matmul(d.kernel_type, a["x1"], a["x2"], a["rhs"], a["params"], a["start"], a["end"])
    assert_close(result, expected)


@pytest.mark.parametrize("variant", ["auto", "block", "mfma_f16_direct", "mfma_f32", "mfma_f32_direct"])
def test_matmul_rhs_dynamic_range(example_data, variant):
    """rhs whose magnitude spans 12 decades across columns and e^24 along the rows: the
    half-precision contraction rescales its operands per column while it walks a row range, so
    results must stay within the usual accumulation bound atol * |K| @ |rhs| everywhere.  The
    half-precision variants represent K / sigma to an absolute 2^-39 (its low half underflows
    below that), which adds the floor 2^-37 * sigma * sum |rhs| over the row's range; it only
    shows when entries of K near zero meet rhs values many decades above the rest.  The
    workgroup-shared variant scales rhs once for four row blocks, so its floor runs over the
    union of their ranges."""
    d = example_data
    n, k = d.rhs.shape[-2], d.rhs.shape[-1]
    col_scale = 10.0 ** torch.linspace(-6, 6, k, device=d.rhs.device)
    if n % 2 == 0:
        row_scale = torch.exp(torch.linspace(-12, 12, n, device=d.rhs.device))
    else:  # odd sizes: magnitude falls along the rows, then jumps back up
        row_scale = torch.exp(-torch.remainder(torch.linspace(0, 48, n, device=d.rhs.device), 24.0) + 12)
    rhs = (d.rhs * col_scale * row_scale[:, None]).contiguous()
    args = (d.x1, d.x2, rhs, d.params, d.start, d.end)
    defines = MatmulSingleConfiguration(d.kernel_type).make_config(args)
    defines["MATMUL_VARIANT"] = variant
    result = load_native("matmul", defines).call(*args).detach().cpu().double().numpy()
    a = d.numpy()
    rhs64 = rhs.detach().cpu().double().numpy()
    kd = oracle.dense(d.kernel_type, a["x1"], a["x2"], a["params"], a["start"], a["end"])
    expected = kd @ rhs64
    if d.kernel_type == "spectral":
        # A phase error of 1e-7 rad (fp32 cosine argument, here or in the reference) changes an
        # entry by that fraction of its Gaussian envelope, not of its own (possibly near-zero)
        # value: the accumulation bound is taken over the envelope.
        env = oracle.dense("rbf", a["x1"], a["x2"], a["params"][..., [0, 2]], a["start"], a["end"])
        bound = np.abs(env) @ np.abs(rhs64)
    else:
        bound = np.abs(kd) @ np.abs(rhs64)
    floor = 0.0
    if variant not in ("mfma_f32", "mfma_f32_direct"):
        start, end = a["start"].copy(), a["end"].copy()
        if variant == "block":
            for g0 in range(0, start.shape[-1], 4):
                s_blk, e_blk = start[..., g0:g0 + 4], end[..., g0:g0 + 4]
                empty = s_blk >= e_blk
                lo = np.where(empty, np.iinfo(np.int32).max, s_blk).min(axis=-1, keepdims=True)
                hi = np.where(empty, 0, e_blk).max(axis=-1, keepdims=True)
                start[..., g0:g0 + 4], end[..., g0:g0 + 4] = np.minimum(lo, hi), hi
        mask = oracle.range_mask(start, end, kd.shape[-2], kd.shape[-1])
        sigma = np.abs(a["params"][..., -1, None, None])
        floor = 2.0 ** -37 * sigma * (mask.astype(np.float64) @ np.abs(rhs64))
    err = np.abs(result - expected)
    assert np.all(np.isfinite(result))
    tol = RTOL * np.abs(expected) + ATOL * bound + floor + 1e-30
    assert np.all(err <= tol), float(np.max(err / tol))


@pytest.mark.square
@pytest.mark.stable
@pytest.mark.parametrize("col_blocks", [1, 2])
def test_matmul_stable(example_data, col_blocks):
    """The reference's `stable` regime (its tests/conftest.py:67-91, 114): evenly spaced x, dense
    pattern, lengthscales of 0.01 ... 0.02."""
    test_matmul(example_data, col_blocks)


@pytest.mark.square
@pytest.mark.stable
@pytest.mark.parametrize("variant,rows", [("valu", None), ("mfma_f32", 128), ("mfma_f16", 32), ("mfma_f16", 128),
                                          ("mfma_f16_direct", 128), ("block", None)])
def test_matmul_variants_stable(example_data, variant, rows):
    test_matmul_variants(example_data, variant, rows)


def _grad_tolerance(expected):
    # Gradients are sums over up to m*n terms of mixed sign: compare relative to the largest
    # component of each batch item's gradient as well as elementwise.
    scale = np.max(np.abs(expected), axis=-1, keepdims=True)
    return ATOL + RTOL * np.maximum(np.abs(expected), scale)


def test_matmul_bwd(example_data):
    d = example_data
    out_grad = torch.randn(*d.params.shape[:-1], d.x1.shape[-1], d.rhs.shape[-1])
    out_grad = (out_grad / torch.linalg.norm(out_grad, dim=(-2, -1), keepdim=True)).to(d.x1.device)
    args = (d.x1, d.x2, d.rhs, d.params, d.start, d.end, out_grad)
    defines = MatmulBwdConfiguration(d.kernel_type).make_config(args)
    result = load_native("matmul_bwd", defines).call(*args)
    a = d.numpy()
    expected = oracle.param_grad(d.kernel_type, a["x1"], a["x2"], out_grad.cpu().numpy(), a["rhs"],
                                 a["params"], a["start"], a["end"])
    err = np.abs(result.cpu().double().numpy() - expected)
    assert np.all(err <= _grad_tolerance(expected)), (result.cpu().numpy(), expected)


def test_bilinear_derivative(example_data):
    d = example_data
    left = torch.randn(*d.x1.shape, 5)
    left = (left / torch.linalg.norm(left, dim=-2, keepdim=True)).to(d.x1.device)
    right = torch.randn(*d.x2.shape, 5)
    right = (right / torch.linalg.norm(right, dim=-2, keepdim=True)).to(d.x1.device)
    args = (d.x1, d.x2, left, right, d.params, d.start, d.end)
    defines = BilinearDerivativeConfiguration(d.kernel_type).make_config(args)
    result = load_native("bilinear_derivative", defines).call(*args)
    a = d.numpy()
    expected = oracle.param_grad(d.kernel_type, a["x1"], a["x2"], left.cpu().numpy(),
                                 right.cpu().numpy(), a["params"], a["start"], a["end"])
    err = np.abs(result.cpu().double().numpy() - expected)
    assert np.all(err <= _grad_tolerance(expected)), (result.cpu().numpy(), expected)


@pytest.mark.square
@pytest.mark.stable
def test_matmul_bwd_stable(example_data):
    test_matmul_bwd(example_data)


@pytest.mark.square
@pytest.mark.stable
def test_bilinear_derivative_stable(example_data):
    test_bilinear_derivative(example_data)


@pytest.mark.square
@pytest.mark.parametrize("shape", [(100,), (5, 101)])
def test_index(example_data, shape):
    d = example_data
    device = d.x1.device
    m, n = d.x1.shape[-1], d.x2.shape[-1]
    batch_indices = tuple(
        torch.randint(0, size, shape, dtype=torch.int32).to(device) for size in d.params.shape[:-1]
    )
    row_index = torch.randint(0, m, shape, dtype=torch.int32).to(device)
    col_index = torch.randint(0, n, shape, dtype=torch.int32).to(device)
    args = (d.x1, d.x2, d.params, d.start, d.end, batch_indices, row_index, col_index)
    defines = IndexConfiguration(d.kernel_type).make_config(args)
    result = load_native("index", defines).call(*args)
    a = d.numpy()
    expected = oracle.index(d.kernel_type, a["x1"], a["x2"], a["params"], a["start"], a["end"],
                            [b.cpu().numpy() for b in batch_indices], row_index.cpu().numpy(),
                            col_index.cpu().numpy())
    assert_close(result, expected)
    # entries outside the pattern are exactly zero
    assert torch.all(result[torch.from_numpy(expected == 0.0).to(device)] == 0.0)


def test_dense(example_data):
    d = example_data
    args = (d.x1, d.x2, d.params, d.start, d.end)
    from kernel_matmul_amd.configurations import DenseConfiguration

    result = load_native("dense", DenseConfiguration(d.kernel_type).make_config(args)).call(*args)
    a = d.numpy()
    expected = oracle.dense(d.kernel_type, a["x1"], a["x2"], a["params"], a["start"], a["end"])
    assert_close(result, expected)
    assert torch.all(result[torch.from_numpy(expected == 0.0).to(result.device)] == 0.0)


def test_dense_bwd(example_data):
    d = example_data
    from kernel_matmul_amd.configurations import DenseBwdConfiguration

    out_grad = torch.randn(*d.params.shape[:-1], d.x1.shape[-1], d.x2.shape[-1])
    out_grad = (out_grad / torch.linalg.norm(out_grad, dim=(-2, -1), keepdim=True)).to(d.x1.device)
    args = (d.x1, d.x2, d.params, d.start, d.end, out_grad)
    result = load_native("dense_bwd", DenseBwdConfiguration(d.kernel_type).make_config(args)).call(*args)
    a = d.numpy()
    grads = oracle.kernel_matrix_grad(d.kernel_type, a["x1"], a["x2"], a["params"])
    mask = oracle.range_mask(a["start"], a["end"], grads.shape[-2], grads.shape[-1])
    weights = np.where(mask, out_grad.cpu().double().numpy(), 0.0)
    expected = np.sum(weights[..., None, :, :] * grads, axis=(-2, -1))
    err = np.abs(result.cpu().double().numpy() - expected)
    assert np.all(err <= _grad_tolerance(expected)), (result.cpu().numpy(), expected)


@pytest.mark.square
@pytest.mark.parametrize("shape", [(100,), (5, 101)])
def test_index_bwd(example_data, shape):
    d = example_data
    from kernel_matmul_amd.configurations import IndexBwdConfiguration

    device = d.x1.device
    m, n = d.x1.shape[-1], d.x2.shape[-1]
    batch_indices = tuple(
        torch.randint(0, size, shape, dtype=torch.int32).to(device) for size in d.params.shape[:-1]
    )
    row_index = torch.randint(0, m, shape, dtype=torch.int32).to(device)
    col_index = torch.clamp(row_index + torch.randint(-40, 40, shape, dtype=torch.int32).to(device), 0, n - 1)
    out_grad = torch.randn(shape).to(device)
    args = (d.x1, d.x2, d.params, d.start, d.end, batch_indices, row_index, col_index, out_grad)
    result = load_native("index_bwd", IndexBwdConfiguration(d.kernel_type).make_config(args)).call(*args)
    a = d.numpy()
    grads = oracle.kernel_matrix_grad(d.kernel_type, a["x1"], a["x2"], a["params"])  # [..., P, m, n]
    mask = oracle.range_mask(a["start"], a["end"], m, n)
    bi = [b.cpu().numpy().astype(np.int64).ravel() for b in batch_indices]
    rows = row_index.cpu().numpy().astype(np.int64).ravel()
    cols = col_index.cpu().numpy().astype(np.int64).ravel()
    og = out_grad.cpu().double().numpy().ravel()
    expected = np.zeros(a["params"].shape, dtype=np.float64)
    for q in range(rows.size):
        b = tuple(x[q] for x in bi)
        if mask[b + (rows[q], cols[q])]:
            expected[b] += og[q] * grads[b + (slice(None), rows[q], cols[q])]
    err = np.abs(result.cpu().double().numpy() - expected)
    assert np.all(err <= _grad_tolerance(expected) + 1e-6), (result.cpu().numpy(), expected)


# Coordinate regimes that decide between the folded evaluation u = fma(x1 - r, s, -(x2 - r) s)
# and the plain (x1 - x2) s inside the split-fp16 kernels: the folded form is only taken where
# both differences are exact in fp32, and either way results must meet the usual tolerance.
COORDINATE_REGIMES = {
    # name: (offset, extent, sorted)
    "offset_1e5": (1.0e5, 150.0, True),      # coarse fp32 grid (ulp 2^-7): differences exact
    "from_zero": (0.0, 150.0, True),         # first point exactly 0: spread > smallest magnitude
    "negative": (-400.0, 150.0, True),       # all negative
    "across_zero": (-75.0, 150.0, True),     # sign change inside the data
    "tiny_offsets": (3.0, 1.0e-3, True),     # everything within one lengthscale
    "unsorted_columns": (10.0, 20.0, False), # x2 in random order, full ranges
}


@pytest.mark.parametrize("variant,k", [("auto", 16), ("block", 16), ("auto", 24), ("mfma_f32", 16), ("mfma_f32", 24)])
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
@pytest.mark.parametrize("regime", sorted(COORDINATE_REGIMES))
def test_matmul_coordinate_regimes(regime, kernel_type, variant, k):
    """k = 24: two groups of rhs columns (the spectral table kernel then takes the cosine per
    entry from tabulated column phases instead of the phase-split form)."""
    from kernel_matmul_amd.ranges import make_ranges
    from tests.conftest import make_params

    offset, extent, is_sorted = COORDINATE_REGIMES[regime]
    g = torch.Generator().manual_seed(11)
    m, batch = 1500, (2,)
    x = torch.rand(m, generator=g) * extent + offset
    if is_sorted:
        x = torch.sort(x)[0]
        if regime == "from_zero":
            x[0] = 0.0
        x1 = x2 = x
        start, end = make_ranges(2.5, x)
    else:
        x1 = torch.sort(x)[0]
        x2 = x[torch.randperm(m, generator=g)]
        rows = (m + 127) // 128
        start = torch.zeros(rows, dtype=torch.int32)
        end = torch.full((rows,), m, dtype=torch.int32)
    rhs = torch.randn(m, k, generator=g)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)  # as the example data does
    params = make_params(kernel_type, batch)
    device = torch.device("cuda:0")
    expand = lambda t: t.to(device).expand(*batch, *t.shape)
    args = (expand(x1), expand(x2), expand(rhs), params.to(device), expand(start), expand(end))
    defines = MatmulSingleConfiguration(kernel_type).make_config(args)
    defines["MATMUL_VARIANT"] = variant
    result = load_native("matmul", defines).call(*args)
    f = lambda t: t.detach().cpu().numpy()
    expected = oracle.matmul(kernel_type, *(f(t) for t in args))
    assert_close(result, expected)


@pytest.mark.parametrize("variant", ["auto", "block", "mfma_f16_direct", "mfma_f32", "mfma_f32_direct", "valu"])
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral"])
def test_matmul_degenerate_ranges(kernel_type, variant):
    """Row blocks with an empty range must produce exact zeros (the output is fully written),
    ranges that reach past the last column are clipped (a symmetric pattern over fewer points
    than one block reports end = block size > n, native/ranges/ranges.cpp:82-93), and single
    rows / columns / rhs columns work."""
    from tests.conftest import make_params

    g = torch.Generator().manual_seed(5)
    device = torch.device("cuda:0")
    for m, n, k, start, end in [
        (300, 300, 3, [0, 120, 290], [50, 120, 400]),   # partial, empty, clipped
        (300, 300, 16, [10, 10, 10], [10, 10, 10]),     # all empty
        (1, 1, 1, [0], [1]),
        (129, 1, 2, [0, 0], [128, 1]),
        (5, 700, 17, [3], [699]),
        # ranges that jump back and forth between neighbouring row blocks, with gaps
        (1000, 1200, 16, [900, 0, 600, 610, 100, 1190, 300, 0], [1200, 40, 900, 611, 500, 1200, 301, 1200]),
    ]:
        x1 = torch.sort(torch.rand(m, generator=g) * 10)[0]
        x2 = torch.sort(torch.rand(n, generator=g) * 10)[0]
        rhs = torch.randn(n, k, generator=g)
        rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)  # as the example data does
        params = make_params(kernel_type, ())
        s = torch.tensor(start, dtype=torch.int32)
        e = torch.tensor(end, dtype=torch.int32)
        args = tuple(t.to(device) for t in (x1, x2, rhs, params, s, e))
        defines = MatmulSingleConfiguration(kernel_type).make_config(args)
        defines["MATMUL_VARIANT"] = variant
        result = load_native("matmul", defines).call(*args)
        f = lambda t: t.detach().cpu().numpy()
        expected = oracle.matmul(kernel_type, *(f(t) for t in args))
        assert_close(result, expected)
        for blk, (lo, hi) in enumerate(zip(start, end)):
            if lo >= hi:
                assert torch.all(result[blk * 128:(blk + 1) * 128] == 0)


@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
def test_param_grad_degenerate_ranges(kernel_type):
    """Same degenerate patterns for the parameter gradient (matmul_bwd)."""
    from tests.conftest import make_params

    g = torch.Generator().manual_seed(6)
    device = torch.device("cuda:0")
    for m, n, k, start, end in [
        (300, 300, 3, [0, 120, 290], [50, 120, 400]),
        (300, 300, 8, [10, 10, 10], [10, 10, 10]),
        (1, 1, 1, [0], [1]),
        (5, 700, 17, [3], [699]),
    ]:
        x1 = torch.sort(torch.rand(m, generator=g) * 10)[0]
        x2 = torch.sort(torch.rand(n, generator=g) * 10)[0]
        rhs = torch.randn(n, k, generator=g)
        out_grad = torch.randn(m, k, generator=g)
        out_grad = out_grad / torch.linalg.norm(out_grad)  # as in test_matmul_bwd
        params = make_params(kernel_type, ())
        s = torch.tensor(start, dtype=torch.int32)
        e = torch.tensor(end, dtype=torch.int32)
        args = tuple(t.to(device) for t in (x1, x2, rhs, params, s, e, out_grad))
        defines = MatmulBwdConfiguration(kernel_type).make_config(args)
        result = load_native("matmul_bwd", defines).call(*args)
        f = lambda t: t.detach().cpu().numpy()
        expected = oracle.param_grad(kernel_type, f(x1), f(x2), f(out_grad), f(rhs), f(params), f(s), f(e))
        err = np.abs(result.cpu().double().numpy() - expected)
        assert np.all(err <= _grad_tolerance(expected)), (result.cpu().numpy(), expected)


@pytest.mark.parametrize("kernel_type", ["rbf", "spectral"])
@pytest.mark.parametrize("n", [1, 8, 63])
def test_bilinear_derivative_narrow_ranges(kernel_type, n):
    """Ranges of a few columns against a row block that spans many lengthscales: nothing averages
    the rounding of a row's sums there, so the gradient must come out at the accuracy of a
    pair-by-pair evaluation, 2e-6 of the sum of |terms| (a form of the gradient that works from
    moments of the row sums reached 7e-5 on a single column; ranges under 64 columns do not take
    it)."""
    g = torch.Generator().manual_seed(31)
    device = torch.device("cuda:0")
    m, c = 127, 5
    for rep in range(4):
        lengthscale = 0.02
        x1 = torch.rand(m, generator=g) * 0.4 + 100.0            # unsorted rows, +-8.5 scaled units
        x2 = torch.sort(torch.rand(n, generator=g) * 0.4 + 100.0)[0]
        cols = [torch.tensor(lengthscale)] + ([torch.tensor(40.6)] if kernel_type == "spectral" else []) + [torch.tensor(1.1)]
        params = torch.stack(cols)
        start = torch.zeros(1, dtype=torch.int32)
        end = torch.full((1,), n, dtype=torch.int32)
        left = torch.randn(m, c, generator=g)
        right = torch.randn(n, c, generator=g)
        args = tuple(t.to(device) for t in (x1, x2, left, right, params, start, end))
        defines = BilinearDerivativeConfiguration(kernel_type).make_config(args)
        result = load_native("bilinear_derivative", defines).call(*args).cpu().double().numpy()
        f = lambda t: t.numpy()
        expected = oracle.param_grad(kernel_type, f(x1), f(x2), f(left), f(right), f(params), f(start), f(end))
        terms = np.abs(oracle.kernel_matrix_grad(kernel_type, f(x1), f(x2), f(params)))
        size = np.sum(np.abs(left.double().numpy() @ right.double().numpy().T)[None] * terms, axis=(-2, -1))
        assert np.all(np.abs(result - expected) <= 2e-6 * size + 1e-9), (result, expected, size)


def _phase_tolerance(kernel_type, a, rhs64, expected, phase_eps):
    """rtol * |expected| + (atol + phase_eps) * (envelope @ |rhs|): a phase error of phase_eps
    radians changes an entry by that fraction of its envelope (the kernel without its
    oscillating factor), in this library and in the reference alike (both form the phase as an
    fp32 product frequency * distance)."""
    if kernel_type == "spectral":
        env = oracle.dense("rbf", a["x1"], a["x2"], a["params"][..., [0, 2]], a["start"], a["end"])
    else:  # locally periodic: |dK/dphase| <= (2 / lp) * sigma * exp(-d^2 / (2 l^2))
        env = oracle.dense("rbf", a["x1"], a["x2"], a["params"][..., [0, 3]], a["start"], a["end"])
        env = env * np.maximum(1.0, 2.0 / np.abs(a["params"][..., 1, None, None]))
    return RTOL * np.abs(expected) + (ATOL + phase_eps) * (np.abs(env) @ np.abs(rhs64)) + 1e-30


@pytest.mark.parametrize("variant", ["auto", "block", "mfma_f16_direct", "mfma_f32", "mfma_f32_direct"])
@pytest.mark.parametrize("frequency", [5.0, 50.0])
def test_matmul_spectral_high_frequency(frequency, variant):
    """Spectral kernels with many oscillations per window (up to 125 revolutions across the
    cutoff) and negative outputscales."""
    from kernel_matmul_amd.ranges import make_ranges

    g = torch.Generator().manual_seed(21)
    m, k, batch = 1500, 16, 3
    x = torch.sort(torch.rand(m, generator=g) * 150.0 + 20.0)[0]
    start, end = make_ranges(2.5, x)
    rhs = torch.randn(m, k, generator=g)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)
    params = torch.stack([1 + torch.rand(batch, generator=g),
                          frequency * (1 + 0.1 * torch.rand(batch, generator=g)),
                          torch.tensor([1.5, -0.7, -2.0])], dim=-1)
    device = torch.device("cuda:0")
    expand = lambda t: t.to(device).expand(batch, *t.shape)
    args = (expand(x), expand(x), expand(rhs), params.to(device), expand(start), expand(end))
    defines = MatmulSingleConfiguration("spectral").make_config(args)
    defines["MATMUL_VARIANT"] = variant
    result = load_native("matmul", defines).call(*args).cpu().double().numpy()
    names = ("x1", "x2", "rhs", "params", "start", "end")
    a = {name: t.detach().cpu().numpy() for name, t in zip(names, args)}
    expected = oracle.matmul("spectral", *(a[name] for name in names))
    # two fp32 roundings of a phase of up to frequency * 1.1 * window revolutions
    window = float((x[end.long().clamp(max=m) - 1] - x[start.long()]).max())
    phase_eps = 2 * np.pi * frequency * 1.1 * window * 2.0 ** -23
    tol = _phase_tolerance("spectral", a, a["rhs"].astype(np.float64), expected, phase_eps)
    err = np.abs(result - expected)
    assert np.all(err <= tol), float(np.max(err / tol))
    assert np.all(np.sign(result[1].sum()) == np.sign(expected[1].sum()))


def _far_phase_problem(kernel_type, k):
    """Long-decay, short-period kernels: the phase frequency * distance reaches thousands of
    revolutions inside the pattern (the hardware sine / cosine only take +-256)."""
    g = torch.Generator().manual_seed(31)
    m, batch = 700, 2
    x = torch.sort(torch.rand(m, generator=g) * 100.0)[0]
    if kernel_type == "spectral":
        params = torch.tensor([[40.0, 30.0, 1.3], [25.0, 47.0, -0.8]])
        revolutions = 47.0 * 100.0
    else:
        params = torch.tensor([[40.0, 1.5, 0.02, 1.3], [25.0, 0.8, 0.011, 0.8]])
        revolutions = 0.5 / 0.011 * 100.0
    rows = (m + 127) // 128
    start = torch.zeros(rows, dtype=torch.int32)
    end = torch.full((rows,), m, dtype=torch.int32)
    rhs = torch.randn(m, k, generator=g)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)
    device = torch.device("cuda:0")
    expand = lambda t: t.to(device).expand(batch, *t.shape)
    t = dict(x=expand(x), rhs=expand(rhs), params=params.to(device), start=expand(start), end=expand(end))
    a = dict(x1=t["x"].cpu().numpy(), x2=t["x"].cpu().numpy(), rhs=t["rhs"].cpu().numpy(),
             params=params.numpy(), start=t["start"].cpu().numpy(), end=t["end"].cpu().numpy())
    phase_eps = 2 * np.pi * revolutions * 2.0 ** -23
    return t, a, phase_eps


@pytest.mark.parametrize("kernel_type", ["spectral", "locally_periodic"])
@pytest.mark.parametrize("variant,k", [("auto", 16), ("auto", 32), ("block", 16), ("mfma_f16_direct", 32),
                                       ("mfma_f32", 16), ("mfma_f32", 32), ("mfma_f32_direct", 16), ("valu", 8)])
def test_matmul_phase_beyond_256_revolutions(kernel_type, variant, k):
    t, a, phase_eps = _far_phase_problem(kernel_type, k)
    args = (t["x"], t["x"], t["rhs"], t["params"], t["start"], t["end"])
    defines = MatmulSingleConfiguration(kernel_type).make_config(args)
    defines["MATMUL_VARIANT"] = variant
    result = load_native("matmul", defines).call(*args).cpu().double().numpy()
    expected = oracle.matmul(kernel_type, a["x1"], a["x2"], a["rhs"], a["params"], a["start"], a["end"])
    tol = _phase_tolerance(kernel_type, a, a["rhs"].astype(np.float64), expected, phase_eps)
    err = np.abs(result - expected)
    assert np.all(err <= tol), float(np.max(err / tol))


@pytest.mark.parametrize("kernel_type", ["spectral", "locally_periodic"])
def test_entry_operators_phase_beyond_256_revolutions(kernel_type):
    """dense, index and the parameter gradient with phases far outside +-256 revolutions."""
    from kernel_matmul_amd.configurations import DenseConfiguration

    t, a, phase_eps = _far_phase_problem(kernel_type, 5)
    device = t["x"].device
    m = a["x1"].shape[-1]
    one = np.ones((m, 1))
    kd = oracle.dense(kernel_type, a["x1"], a["x2"], a["params"], a["start"], a["end"])
    dense_args = (t["x"], t["x"], t["params"], t["start"], t["end"])
    got = load_native("dense", DenseConfiguration(kernel_type).make_config(dense_args)).call(*dense_args)
    # per entry: the tolerance of a product with a one-hot rhs
    if kernel_type == "spectral":
        env = oracle.dense("rbf", a["x1"], a["x2"], a["params"][..., [0, 2]], a["start"], a["end"])
    else:
        env = oracle.dense("rbf", a["x1"], a["x2"], a["params"][..., [0, 3]], a["start"], a["end"])
        env = env * np.maximum(1.0, 2.0 / np.abs(a["params"][..., 1, None, None]))
    tol = RTOL * np.abs(kd) + (ATOL + phase_eps) * np.abs(env)
    err = np.abs(got.cpu().double().numpy() - kd)
    assert np.all(err <= tol), float(np.max(err / np.maximum(tol, 1e-30)))

    gen = torch.Generator().manual_seed(32)
    q = 500
    rows = torch.randint(0, m, (q,), generator=gen, dtype=torch.int32)
    cols = torch.randint(0, m, (q,), generator=gen, dtype=torch.int32)
    bi = torch.randint(0, 2, (q,), generator=gen, dtype=torch.int32)
    iargs = (t["x"], t["x"], t["params"], t["start"], t["end"], (bi.to(device),), rows.to(device), cols.to(device))
    igot = load_native("index", IndexConfiguration(kernel_type).make_config(iargs)).call(*iargs)
    sel = (bi.numpy().astype(np.int64), rows.numpy().astype(np.int64), cols.numpy().astype(np.int64))
    ierr = np.abs(igot.cpu().double().numpy() - kd[sel])
    assert np.all(ierr <= tol[sel]), float(np.max(ierr / np.maximum(tol[sel], 1e-30)))

    left = torch.randn(2, m, 5, generator=gen)
    left = (left / torch.linalg.norm(left, dim=-2, keepdim=True)).to(device)
    gargs = (t["x"], t["x"], left, t["rhs"], t["params"], t["start"], t["end"])
    ggot = load_native("bilinear_derivative",
                       BilinearDerivativeConfiguration(kernel_type).make_config(gargs)).call(*gargs)
    gexp = oracle.param_grad(kernel_type, a["x1"], a["x2"], left.cpu().numpy(), a["rhs"], a["params"],
                             a["start"], a["end"])
    # bound of the phase error's effect: sum over pairs of |coefficient| * |d(dK/dtheta)/dphase|;
    # taken as the sum of |coefficient * dK/dtheta| scaled up by the largest phase sensitivity
    grads = oracle.kernel_matrix_grad(kernel_type, a["x1"], a["x2"], a["params"])
    coeff = np.abs(left.cpu().double().numpy() @ np.swapaxes(a["rhs"].astype(np.float64), -1, -2))
    envg = oracle.kernel_matrix_grad("rbf", a["x1"], a["x2"], a["params"][..., [0, -1]])
    env_l = np.sum(coeff * np.abs(envg[..., 0, :, :]), axis=(-2, -1))
    env_s = np.sum(coeff * np.abs(envg[..., 1, :, :]), axis=(-2, -1))
    dmax = 100.0
    sig = np.abs(a["params"][..., -1])
    if kernel_type == "spectral":
        f = a["params"][..., 1]
        bound = np.stack([env_l, 2 * np.pi * dmax * sig * env_s * (1 + 0 * f), env_s], axis=-1)
    else:
        lp, T = a["params"][..., 1], a["params"][..., 2]
        amp = np.maximum(1.0, 2.0 / lp)
        bound = np.stack([env_l * amp, 2 / lp**2 * sig * env_s * amp,
                          4 * np.pi * dmax / (lp * T**2) * sig * env_s * amp, env_s * amp], axis=-1)
    gerr = np.abs(ggot.cpu().double().numpy() - gexp)
    gtol = _grad_tolerance(gexp) + 4 * phase_eps * bound
    assert np.all(gerr <= gtol), (ggot.cpu().numpy(), gexp, gerr / gtol)
    del one


# The parameter gradient takes a feature form (moments of the columns about a reference point
# per wavefront) only where that loses nothing and redoes the other row blocks pair by pair:
# exact coordinate differences, rows within 12 and columns within 48 scaled lengths of the
# reference point.  Every regime must meet the tolerance, whichever form its row blocks take.
GRADIENT_REGIMES = dict(COORDINATE_REGIMES)
GRADIENT_REGIMES.update({
    "sparse_rows": (50.0, 6000.0, True),     # a row block spans hundreds of lengthscales
    "dense_rows": (50.0, 15.0, True),        # everything within a few lengthscales
})


@pytest.mark.parametrize("vector_width", [3, 5, 8])
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
@pytest.mark.parametrize("regime", sorted(GRADIENT_REGIMES))
def test_param_grad_coordinate_regimes(regime, kernel_type, vector_width):
    from kernel_matmul_amd.ranges import make_ranges
    from tests.conftest import make_params

    offset, extent, is_sorted = GRADIENT_REGIMES[regime]
    g = torch.Generator().manual_seed(12)
    m, batch = 1500, (2,)
    x = torch.rand(m, generator=g) * extent + offset
    if is_sorted:
        x = torch.sort(x)[0]
        if regime == "from_zero":
            x[0] = 0.0
        x1 = x2 = x
        start, end = make_ranges(2.5 if extent < 1000 else 12.0, x)
    else:
        x1 = torch.sort(x)[0]
        x2 = x[torch.randperm(m, generator=g)]
        rows = (m + 127) // 128
        start = torch.zeros(rows, dtype=torch.int32)
        end = torch.full((rows,), m, dtype=torch.int32)
    left = torch.randn(*batch, m, vector_width, generator=g)
    left = left / torch.linalg.norm(left, dim=-2, keepdim=True)
    right = torch.randn(m, vector_width, generator=g)
    right = right / torch.linalg.norm(right, dim=-2, keepdim=True)
    params = make_params(kernel_type, batch)
    device = torch.device("cuda:0")
    expand = lambda t: t.to(device).expand(*batch, *t.shape)
    args = (expand(x1), expand(x2), left.to(device), expand(right), params.to(device), expand(start), expand(end))
    result = load_native("bilinear_derivative",
                         BilinearDerivativeConfiguration(kernel_type).make_config(args)).call(*args)
    f = lambda t: t.detach().cpu().numpy()
    expected = oracle.param_grad(kernel_type, *(f(t) for t in args))
    err = np.abs(result.cpu().double().numpy() - expected)
    assert np.all(err <= _grad_tolerance(expected)), (result.cpu().numpy(), expected)


@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
def test_index_bwd_blocks_of_one_and_of_several_batch_items(kernel_type):
    """The diagonal of a batch of matrices as index entries (batch-major, 700 entries per item):
    blocks of 256 entries that lie inside one batch item go through their block sums, the blocks
    across an item boundary entry by entry; a second call with the items interleaved entry by
    entry has no uniform block at all.  Both against the float64 oracle."""
    from kernel_matmul_amd.configurations import IndexBwdConfiguration
    from kernel_matmul_amd.ranges import make_ranges
    from tests.conftest import make_params

    device = torch.device("cuda:0")
    nb, n = 3, 700
    x = torch.sort(torch.rand(n) * 10)[0]
    params = make_params(kernel_type, (nb,))
    start, end = make_ranges(2.0, x)
    grads = oracle.kernel_matrix_grad(kernel_type, x.numpy(), x.numpy(), params.numpy())  # [nb, P, n, n]
    mask = oracle.range_mask(start.numpy(), end.numpy(), n, n)
    xb, sb, eb = x.to(device).expand(nb, n), start.to(device).expand(nb, -1), end.to(device).expand(nb, -1)
    for interleaved in (False, True):
        if interleaved:
            bi = (torch.arange(nb * n, dtype=torch.int32) % nb).reshape(n, nb)
            ri = (torch.arange(nb * n, dtype=torch.int32) // nb).reshape(n, nb)
        else:
            bi = torch.arange(nb, dtype=torch.int32)[:, None].expand(nb, n).contiguous()
            ri = torch.arange(n, dtype=torch.int32)[None, :].expand(nb, n).contiguous()
        ci = torch.clamp(ri + 3, max=n - 1)
        og = torch.randn(bi.shape)
        args = (xb, xb, params.to(device), sb, eb, (bi.to(device),), ri.to(device), ci.to(device), og.to(device))
        result = load_native("index_bwd", IndexBwdConfiguration(kernel_type).make_config(args)).call(*args)
        expected = np.zeros(params.shape, dtype=np.float64)
        b_, r_, c_, g_ = (t.numpy().ravel() for t in (bi, ri, ci, og.double()))
        for q in range(b_.size):
            if mask[r_[q], c_[q]]:
                expected[b_[q]] += g_[q] * grads[b_[q], :, r_[q], c_[q]]
        err = np.abs(result.cpu().double().numpy() - expected)
        assert np.all(err <= _grad_tolerance(expected) + 1e-6), (interleaved, result.cpu().numpy(), expected)
