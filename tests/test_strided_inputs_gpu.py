"""Inputs that are views with non-unit or padded inner strides.

The reference addresses every tensor through its strides (native/common/accessor.cuh:12-56), so a
caller may hand over a transposed rhs, a column slice of a wider matrix, every second element of
a longer coordinate vector or hyper-parameters cut out of a larger tensor.  Each case here runs an
operator on such views and on plain contiguous copies of the same values; matmul and the
parameter gradients are compared with the float64 oracle, the entry operators with their own
result on the contiguous copies (which tests/test_ops_gpu.py pins to the oracle).  The gaps of the
views hold NaN (floats) or a large negative number (ranges), so a load that ignores a stride shows.

Tolerances as in tests/test_ops_gpu.py: rtol 1e-4 / atol 1e-5 (gradients relative to their scale).
"""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.compile import load_native
from kernel_matmul_amd.configurations import (
    BilinearDerivativeConfiguration,
    DenseBwdConfiguration,
    DenseConfiguration,
    IndexBwdConfiguration,
    IndexConfiguration,
    MatmulSingleConfiguration,
)
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle
from tests.conftest import KERNEL_TYPES, make_params

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5
DEVICE = torch.device("cuda:0")


def _gap_value(t):
    return float("nan") if t.is_floating_point() else -(2 ** 30)


def interleaved(t):
    """Same values at stride 2 along the last dimension."""
    big = torch.full((*t.shape[:-1], 2 * t.shape[-1]), _gap_value(t), dtype=t.dtype, device=t.device)
    big[..., ::2] = t
    view = big[..., ::2]
    assert view.stride(-1) == 2 or t.shape[-1] == 1
    return view


def padded(t, before=2, after=3):
    """Same values as a slice of a wider last dimension."""
    n = t.shape[-1]
    big = torch.full((*t.shape[:-1], before + n + after), _gap_value(t), dtype=t.dtype, device=t.device)
    big[..., before:before + n] = t
    view = big[..., before:before + n]
    assert view.storage_offset() == before and view.data_ptr() != big.data_ptr()
    return view


def column_major(t):
    """Same matrix with the second-to-last dimension contiguous."""
    view = t.transpose(-1, -2).contiguous().transpose(-1, -2)
    assert view.stride(-2) == 1 or t.shape[-2] == 1
    return view


def make_case(kernel_type, m, n, k, batch, seed):
    g = torch.Generator().manual_seed(seed)
    x1 = torch.sort(torch.rand(*batch, m, generator=g) * 10, dim=-1)[0]
    x2 = torch.sort(torch.rand(*batch, n, generator=g) * 10, dim=-1)[0]
    start, end = make_ranges(2.0, x1, x2)
    rhs = torch.randn(*batch, n, k, generator=g)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)
    params = make_params(kernel_type, batch)
    return dict(x1=x1, x2=x2, rhs=rhs, params=params, start=start.contiguous(), end=end.contiguous())


def to_device(case):
    return {name: t.to(DEVICE) for name, t in case.items()}


def as_numpy(case):
    return {name: t.detach().cpu().numpy() for name, t in case.items()}


# name -> {tensor name: layout function}
MATMUL_LAYOUTS = {
    "column_major_rhs": dict(rhs=column_major),
    "rhs_columns_of_a_wider_matrix": dict(rhs=padded),
    "interleaved_coordinates": dict(x1=interleaved, x2=interleaved),
    "interleaved_ranges": dict(start=interleaved, end=interleaved),
    "params_slice": dict(params=padded),
    "everything": dict(x1=padded, x2=interleaved, rhs=column_major, params=padded, start=interleaved,
                       end=padded),
}


def apply_layout(tensors, layout):
    return {name: layout.get(name, lambda t: t)(t) for name, t in tensors.items()}


def assert_close(actual, expected, tol=None):
    actual = actual.detach().cpu().double().numpy()
    assert actual.shape == expected.shape
    err = np.abs(actual - expected)
    tol = ATOL + RTOL * np.abs(expected) if tol is None else tol
    assert np.all(err <= tol), f"max error {np.nanmax(err):.3e}, NaNs: {int(np.isnan(actual).sum())}"


def grad_tolerance(expected):
    scale = np.max(np.abs(expected), axis=-1, keepdims=True)
    return ATOL + RTOL * np.maximum(np.abs(expected), scale)


@pytest.mark.parametrize("variant,k", [("auto", 1), ("auto", 16), ("auto", 24), ("auto", 65), ("block", 16),
                                       ("mfma_f32", 16), ("mfma_f32_direct", 24), ("mfma_f16_direct", 16),
                                       ("valu", 11)])
@pytest.mark.parametrize("layout", sorted(MATMUL_LAYOUTS))
@pytest.mark.parametrize("kernel_type", KERNEL_TYPES)
def test_matmul_with_strided_views(kernel_type, layout, variant, k):
    case = make_case(kernel_type, 600, 800, k, (2,), seed=5)
    expected = oracle.matmul(kernel_type, *(as_numpy(case)[name] for name in
                                            ("x1", "x2", "rhs", "params", "start", "end")))
    views = apply_layout(to_device(case), MATMUL_LAYOUTS[layout])
    args = tuple(views[name] for name in ("x1", "x2", "rhs", "params", "start", "end"))
    defines = MatmulSingleConfiguration(kernel_type).make_config(args)
    defines["MATMUL_VARIANT"] = variant
    result = load_native("matmul", defines).call(*args)
    assert result.is_contiguous()
    assert_close(result, expected)


GRAD_LAYOUTS = {
    "column_major_vectors": dict(left=column_major, right=column_major),
    "vector_columns_of_wider_matrices": dict(left=padded, right=padded),
    "interleaved_coordinates_and_ranges": dict(x1=interleaved, x2=interleaved, start=interleaved,
                                               end=interleaved),
    "everything": dict(x1=interleaved, x2=padded, left=padded, right=column_major, params=padded,
                       start=padded, end=interleaved),
}


@pytest.mark.parametrize("width", [3, 8])   # feature form (rbf, spectral) / pairwise form
@pytest.mark.parametrize("layout", sorted(GRAD_LAYOUTS))
@pytest.mark.parametrize("kernel_type", KERNEL_TYPES)
def test_bilinear_derivative_with_strided_views(kernel_type, layout, width):
    case = make_case(kernel_type, 700, 700, width, (2,), seed=6)
    g = torch.Generator().manual_seed(7)
    left = torch.randn(2, 700, width, generator=g)
    case["left"] = left / torch.linalg.norm(left, dim=-2, keepdim=True)
    case["right"] = case.pop("rhs")
    a = as_numpy(case)
    expected = oracle.param_grad(kernel_type, a["x1"], a["x2"], a["left"], a["right"], a["params"],
                                 a["start"], a["end"])
    views = apply_layout(to_device(case), GRAD_LAYOUTS[layout])
    args = tuple(views[name] for name in ("x1", "x2", "left", "right", "params", "start", "end"))
    defines = BilinearDerivativeConfiguration(kernel_type).make_config(args)
    result = load_native("bilinear_derivative", defines).call(*args)
    assert_close(result, expected, grad_tolerance(expected))


ENTRY_LAYOUT = dict(x1=interleaved, x2=padded, params=padded, start=interleaved, end=padded)


@pytest.mark.parametrize("kernel_type", KERNEL_TYPES)
def test_entry_operators_with_strided_views(kernel_type):
    """index, dense and their gradients: same results from views as from contiguous copies."""
    case = make_case(kernel_type, 300, 300, 1, (3,), seed=8)
    case.pop("rhs")
    plain = to_device(case)
    views = apply_layout(plain, ENTRY_LAYOUT)
    g = torch.Generator().manual_seed(9)
    count = 500
    batch_index = torch.randint(0, 3, (count,), generator=g, dtype=torch.int32)
    row_index = torch.randint(0, 300, (count,), generator=g, dtype=torch.int32)
    col_index = torch.clamp(row_index + torch.randint(-30, 30, (count,), generator=g, dtype=torch.int32), 0, 299)
    entry_grad = torch.randn(count, generator=g)
    dense_grad = torch.randn(3, 300, 300, generator=g)
    index_plain = tuple(t.to(DEVICE) for t in (batch_index, row_index, col_index))
    index_views = tuple(interleaved(t) for t in index_plain)

    def run(op, configuration, tensors, *extra):
        args = tuple(tensors[name] for name in ("x1", "x2", "params", "start", "end")) + extra
        return load_native(op, configuration(kernel_type).make_config(args)).call(*args)

    for op, configuration, extra_plain, extra_views in [
        ("dense", DenseConfiguration, (), ()),
        ("dense_bwd", DenseBwdConfiguration, (dense_grad.to(DEVICE),),
         (column_major(dense_grad.to(DEVICE)),)),
        ("index", IndexConfiguration, ((index_plain[0],), index_plain[1], index_plain[2]),
         ((index_views[0],), index_views[1], index_views[2])),
        ("index_bwd", IndexBwdConfiguration,
         ((index_plain[0],), index_plain[1], index_plain[2], entry_grad.to(DEVICE)),
         ((index_views[0],), index_views[1], index_views[2], interleaved(entry_grad.to(DEVICE)))),
    ]:
        expected = run(op, configuration, plain, *extra_plain).cpu().double().numpy()
        result = run(op, configuration, views, *extra_views)
        assert np.all(np.isfinite(expected)), op
        tol = grad_tolerance(expected) if op.endswith("_bwd") else None
        assert_close(result, expected, tol)


LARGEST_STRIDE = 1 << 22


@pytest.mark.parametrize("variant,k", [("auto", 16), ("auto", 24), ("mfma_f32", 16), ("mfma_f16_direct", 64)])
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral"])
def test_matmul_at_the_largest_inner_strides(kernel_type, variant, k):
    """rhs rows 2^22 elements apart, x2 elements 2^22 apart, and rhs columns 2^22 apart: the
    kernels' 32-bit byte offsets at the limit the entry point accepts."""
    n = 200
    case = make_case(kernel_type, 300, n, k, (), seed=10)
    expected = oracle.matmul(kernel_type, *(as_numpy(case)[name] for name in
                                            ("x1", "x2", "rhs", "params", "start", "end")))
    plain = to_device(case)
    store = torch.empty(n * LARGEST_STRIDE, device=DEVICE)

    def spread(t, strides):
        view = store.as_strided(tuple(t.shape), strides)
        view.copy_(t)
        return view

    for name, strides in [("rhs", (LARGEST_STRIDE, 1)), ("rhs", (1, LARGEST_STRIDE)), ("x2", (LARGEST_STRIDE,))]:
        tensors = dict(plain)
        tensors[name] = spread(plain[name], strides)
        args = tuple(tensors[key] for key in ("x1", "x2", "rhs", "params", "start", "end"))
        defines = MatmulSingleConfiguration(kernel_type).make_config(args)
        defines["MATMUL_VARIANT"] = variant
        assert_close(load_native("matmul", defines).call(*args), expected)
    del store


def test_matmul_rejects_inner_strides_beyond_the_limit():
    case = to_device(make_case("rbf", 300, 64, 4, (), seed=11))
    store = torch.zeros(64 * (LARGEST_STRIDE + 1), device=DEVICE)
    case["rhs"] = store.as_strided((64, 4), (LARGEST_STRIDE + 1, 1))
    args = tuple(case[key] for key in ("x1", "x2", "rhs", "params", "start", "end"))
    defines = MatmulSingleConfiguration("rbf").make_config(args)
    with pytest.raises(RuntimeError, match="inner strides"):
        load_native("matmul", defines).call(*args)


@pytest.mark.parametrize("kernel_type", ["rbf", "spectral"])
def test_bilinear_derivative_with_strides_beyond_the_feature_form(kernel_type):
    """Inner strides above 2^24 elements: the narrow-vector form's 32-bit offsets do not reach,
    and the library evaluates pair by pair instead of refusing."""
    stride = (1 << 24) + 1
    n, width = 150, 3
    case = make_case(kernel_type, 300, n, width, (), seed=12)
    g = torch.Generator().manual_seed(13)
    left = torch.randn(300, width, generator=g)
    case["left"] = left / torch.linalg.norm(left, dim=-2, keepdim=True)
    case["right"] = case.pop("rhs")
    a = as_numpy(case)
    expected = oracle.param_grad(kernel_type, a["x1"], a["x2"], a["left"], a["right"], a["params"],
                                 a["start"], a["end"])
    plain = to_device(case)
    store = torch.empty(n * stride, device=DEVICE)
    for name, strides in [("right", (stride, 1)), ("x2", (stride,))]:
        tensors = dict(plain)
        view = store.as_strided(tuple(plain[name].shape), strides)
        view.copy_(plain[name])
        tensors[name] = view
        args = tuple(tensors[key] for key in ("x1", "x2", "left", "right", "params", "start", "end"))
        defines = BilinearDerivativeConfiguration(kernel_type).make_config(args)
        result = load_native("bilinear_derivative", defines).call(*args)
        assert_close(result, expected, grad_tolerance(expected))
    del store
