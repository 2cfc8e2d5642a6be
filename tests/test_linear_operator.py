"""KernelMatmulLinearOperator: argument validation on the CPU, operator algebra and autograd
against the float64 oracle on the GPU (reference: tests/test_linear_operator.py,
kernel_matmul/linear_operator.py:88-289)."""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.linear_operator import KernelMatmulLinearOperator
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle


def test_constructor_validation():
    x = torch.zeros(10, 1)
    params = torch.ones(2)
    start = torch.zeros(1, dtype=torch.int32)
    end = torch.full((1,), 10, dtype=torch.int32)
    with pytest.raises(ValueError, match="kernel_type must be specified"):
        KernelMatmulLinearOperator(x, x, params, start, end)
    with pytest.raises(ValueError, match=r"x1 and x2 must have shapes"):
        KernelMatmulLinearOperator(x.squeeze(-1), x, params, start, end, kernel_type="rbf")
    with pytest.raises(ValueError, match=r"x1 and x2 must have shapes"):
        KernelMatmulLinearOperator(x, torch.zeros(10, 2), params, start, end, kernel_type="rbf")


def test_shape_broadcast_and_dtype_device_refusal():
    x = torch.sort(torch.rand(300, 1), dim=0)[0]
    params = torch.ones(4, 2)
    start, end = make_ranges(1.0, x.squeeze(-1))
    op = KernelMatmulLinearOperator(x, x, params, start, end, kernel_type="rbf")
    assert op.shape == torch.Size((4, 300, 300))
    assert op._x1.stride(0) == 0 and op._start.stride(0) == 0  # expanded views, no copies
    assert op._symmetric is True
    assert op._transpose_nonbatch() is op
    with pytest.raises(NotImplementedError, match="only supports CUDA and float32"):
        op.to(torch.device("cpu"))
    with pytest.raises(NotImplementedError, match="only supports CUDA and float32"):
        op.to(torch.float64)
    with pytest.raises(NotImplementedError, match="only supports CUDA and float32"):
        op.type(torch.float64)
    wider = op._expand_batch(torch.Size((2, 4)))
    assert wider.shape == torch.Size((2, 4, 300, 300))


def test_widened_constructor_tensors_are_views_kept_for_the_last_batch_shape():
    x = torch.sort(torch.rand(300, 1), dim=0)[0]
    params = torch.ones(4, 2)
    start, end = make_ranges(1.0, x.squeeze(-1))
    op = KernelMatmulLinearOperator(x, x, params, start, end, kernel_type="rbf")
    first = op._get_args_for_native(torch.Size((4,)))
    second = op._get_args_for_native((4,))
    assert all(t is s for t, s in zip(first, second))
    assert all(t.untyped_storage().data_ptr() == s.untyped_storage().data_ptr()
               for t, s in zip(first, (x, x, params, start, end)))
    wider = op._get_args_for_native((2, 4))
    assert wider[0] is not first[0] and wider[2].shape == (2, 4, 2) and wider[2].stride(0) == 0
    again = op._get_args_for_native((4,))
    assert [t.shape for t in again] == [t.shape for t in first]


def test_widened_params_follow_the_autograd_mode_of_each_call():
    """A first call under no_grad (or inference_mode) must not cut later calls off from the
    hyper-parameters: the widened view of params is made per call, only the gradient-free
    tensors are kept."""
    x = torch.sort(torch.rand(300, 1), dim=0)[0]
    start, end = make_ranges(1.0, x.squeeze(-1))
    for first_mode in (torch.no_grad, torch.inference_mode):
        params = torch.ones(2, requires_grad=True)
        op = KernelMatmulLinearOperator(x, x, params, start, end, kernel_type="rbf")
        for shape in ((), (3,)):
            with first_mode():
                quiet = op._get_args_for_native(shape)
            live = op._get_args_for_native(shape)
            assert live[2].requires_grad and not live[2].is_inference()
            assert shape == () or live[2].grad_fn is not None  # () is the operator's own shape: no new view
            assert live[0] is quiet[0] and live[3] is quiet[3]
            params.grad = None
            (live[2] * torch.arange(1.0, 3.0)).sum().backward()
            assert torch.equal(params.grad, torch.arange(1.0, 3.0) * max(1, int(np.prod(shape))))


def _make_operator(kernel_type, batch, m, n, device, square, requires_grad=False):
    g = torch.Generator().manual_seed(17)
    x1 = torch.sort(torch.rand(m, generator=g) * 10)[0]
    x2 = x1 if square else torch.sort(torch.rand(n, generator=g) * 10)[0]
    p = {"rbf": 2, "spectral": 3, "locally_periodic": 4}[kernel_type]
    params = 0.6 + torch.rand(*batch, p, generator=g)
    start, end = (make_ranges(2.0, x1, align=True) if square else make_ranges(2.0, x1, x2, align=True))
    params = params.to(device).requires_grad_(requires_grad)
    op = KernelMatmulLinearOperator(
        x1.to(device).unsqueeze(-1), x2.to(device).unsqueeze(-1), params, start.to(device),
        end.to(device), kernel_type=kernel_type, symmetric=square,
    )
    arrays = dict(x1=x1.numpy(), x2=x2.numpy(), params=params.detach().cpu().numpy(),
                  start=start.numpy(), end=end.numpy())
    return op, params, arrays


def _dense(kernel_type, a, batch):
    bc = lambda v: np.broadcast_to(v, (*batch, *v.shape))
    return oracle.dense(kernel_type, bc(a["x1"]), bc(a["x2"]), a["params"], bc(a["start"]), bc(a["end"]))


@pytest.mark.gpu
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
@pytest.mark.parametrize("square", [True, False])
def test_matmul_transpose_dense_diagonal(kernel_type, square):
    device = torch.device("cuda:0")
    batch, m, n = (3,), 400, (400 if square else 333)
    op, _, a = _make_operator(kernel_type, batch, m, n, device, square)
    dense = _dense(kernel_type, a, batch)
    rhs = torch.randn(n, 5)
    out = op._matmul(rhs.to(device))
    assert out.shape == (3, m, 5)
    np.testing.assert_allclose(out.cpu().numpy(), dense @ rhs.double().numpy(), rtol=1e-4, atol=1e-5)
    vec = op.matmul(rhs[:, 0].to(device)) if hasattr(op, "matmul") else None
    if vec is not None:
        np.testing.assert_allclose(vec.cpu().numpy(), (dense @ rhs[:, :1].double().numpy())[..., 0], rtol=1e-4, atol=1e-5)

    op_t = op._transpose_nonbatch()
    assert op_t.shape == (3, n, m)
    rhs_t = torch.randn(3, m, 2)
    out_t = op_t._matmul(rhs_t.to(device))
    np.testing.assert_allclose(out_t.cpu().numpy(), np.swapaxes(dense, -1, -2) @ rhs_t.double().numpy(),
                               rtol=1e-4, atol=1e-5)

    np.testing.assert_allclose(op.to_dense().cpu().numpy(), dense, rtol=1e-4, atol=1e-5)
    if square:
        diag = op.diagonal()
        np.testing.assert_allclose(diag.cpu().numpy(), np.diagonal(dense, axis1=-2, axis2=-1), rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
@pytest.mark.parametrize("square", [True, False])
def test_autograd_params_and_rhs(kernel_type, square):
    device = torch.device("cuda:0")
    batch, m, n = (2,), 300, (300 if square else 270)
    op, params, a = _make_operator(kernel_type, batch, m, n, device, square, requires_grad=True)
    rhs = torch.randn(2, n, 4, device=device, requires_grad=True)
    weight = torch.randn(2, m, 4, device=device)
    (op._matmul(rhs) * weight).sum().backward()

    bc = lambda v: np.broadcast_to(v, (*batch, *v.shape))
    expected_params = oracle.param_grad(kernel_type, bc(a["x1"]), bc(a["x2"]), weight.cpu().numpy(),
                                        rhs.detach().cpu().numpy(), a["params"], bc(a["start"]), bc(a["end"]))
    scale = np.abs(expected_params).max(axis=-1, keepdims=True)
    assert np.all(np.abs(params.grad.cpu().numpy() - expected_params) <= 1e-5 + 1e-4 * scale)
    dense = _dense(kernel_type, a, batch)
    expected_rhs = np.swapaxes(dense, -1, -2) @ weight.cpu().double().numpy()
    np.testing.assert_allclose(rhs.grad.cpu().numpy(), expected_rhs, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_params_gradient_after_a_first_call_without_grad():
    device = torch.device("cuda:0")
    op, params, a = _make_operator("spectral", (2,), 300, 300, device, True, requires_grad=True)
    rhs = torch.randn(2, 300, 4, device=device)
    weight = torch.randn(2, 300, 4, device=device)
    with torch.no_grad():
        quiet = op._matmul(rhs)
    out = op._matmul(rhs)
    assert torch.equal(out, quiet)
    (out * weight).sum().backward()
    bc = lambda v: np.broadcast_to(v, (2, *v.shape))
    expected = oracle.param_grad("spectral", bc(a["x1"]), bc(a["x2"]), weight.cpu().numpy(), rhs.cpu().numpy(),
                                 a["params"], bc(a["start"]), bc(a["end"]))
    scale = np.abs(expected).max(axis=-1, keepdims=True)
    assert params.grad is not None
    assert np.all(np.abs(params.grad.cpu().numpy() - expected) <= 1e-5 + 1e-4 * scale)


@pytest.mark.gpu
def test_matmul_rhs_batch_shapes_in_turn():
    """rhs with the operator's batch shape (no broadcast needed), with none, with a wider one,
    and the first again: each call widens the constructor tensors for its own shape."""
    device = torch.device("cuda:0")
    op, _, a = _make_operator("spectral", (3,), 400, 400, device, True)
    dense = _dense("spectral", a, (3,))
    g = torch.Generator().manual_seed(5)
    for shape in [(3, 400, 4), (400, 4), (2, 3, 400, 4), (1, 400, 4), (3, 400, 4)]:
        rhs = torch.randn(*shape, generator=g)
        out = op._matmul(rhs.to(device))
        expected = dense @ rhs.double().numpy()
        assert out.shape == expected.shape
        np.testing.assert_allclose(out.cpu().numpy(), expected, rtol=1e-4, atol=1e-5)
    diag = op.diagonal()
    np.testing.assert_allclose(diag.cpu().numpy(), np.diagonal(dense, axis1=-2, axis2=-1), rtol=1e-5)
    np.testing.assert_allclose(op.diagonal().cpu().numpy(), diag.cpu().numpy(), rtol=0)


@pytest.mark.gpu
def test_bilinear_derivative_hook():
    device = torch.device("cuda:0")
    op, params, a = _make_operator("spectral", (2,), 300, 300, device, True)
    left = torch.randn(300, 3, device=device)
    right = torch.randn(2, 300, 3, device=device)
    grads = op._bilinear_derivative(left, right)
    assert len(grads) == 5 and grads[0] is None and grads[1] is None and grads[3] is None
    bc = lambda v: np.broadcast_to(v, (2, *v.shape))
    expected = oracle.param_grad("spectral", bc(a["x1"]), bc(a["x2"]), bc(left.cpu().numpy()),
                                 right.cpu().numpy(), a["params"], bc(a["start"]), bc(a["end"]))
    scale = np.abs(expected).max(axis=-1, keepdims=True)
    assert grads[2].shape == (2, 3)
    assert np.all(np.abs(grads[2].cpu().numpy() - expected) <= 1e-5 + 1e-4 * scale)


@pytest.mark.gpu
def test_rhs_gradient_needs_aligned_pattern():
    device = torch.device("cuda:0")
    x1 = torch.sort(torch.rand(300) * 10)[0]
    x2 = torch.sort(torch.rand(280) * 10)[0]
    start, end = make_ranges(1.0, x1, x2, align=False)
    op = KernelMatmulLinearOperator(x1.to(device)[:, None], x2.to(device)[:, None],
                                    torch.ones(2, device=device), start.to(device), end.to(device),
                                    kernel_type="rbf")
    rhs = torch.randn(280, 2, device=device, requires_grad=True)
    with pytest.raises(RuntimeError, match="align=True"):
        op._matmul(rhs).sum().backward()


@pytest.mark.gpu
@pytest.mark.parametrize("kernel_type", ["rbf", "spectral", "locally_periodic"])
def test_autograd_through_to_dense_and_diagonal(kernel_type):
    device = torch.device("cuda:0")
    batch = (2,)
    op, params, a = _make_operator(kernel_type, batch, 300, 300, device, True, requires_grad=True)
    weight = torch.randn(2, 300, 300, device=device)
    (op.to_dense() * weight).sum().backward()
    bc = lambda v: np.broadcast_to(v, (*batch, *v.shape))
    grads = oracle.kernel_matrix_grad(kernel_type, bc(a["x1"]), bc(a["x2"]), a["params"])
    mask = oracle.range_mask(bc(a["start"]), bc(a["end"]), 300, 300)
    expected = np.sum(np.where(mask, weight.cpu().double().numpy(), 0.0)[..., None, :, :] * grads, axis=(-2, -1))
    scale = np.abs(expected).max(axis=-1, keepdims=True)
    assert np.all(np.abs(params.grad.cpu().numpy() - expected) <= 1e-5 + 1e-4 * scale)

    params.grad = None
    dweight = torch.randn(2, 300, device=device)
    (op.diagonal() * dweight).sum().backward()
    diag_grads = np.diagonal(grads, axis1=-2, axis2=-1)  # [b, P, n]
    expected = np.sum(diag_grads * dweight.cpu().double().numpy()[:, None, :], axis=-1)
    scale = np.abs(expected).max(axis=-1, keepdims=True)
    assert np.all(np.abs(params.grad.cpu().numpy() - expected) <= 1e-5 + 1e-4 * scale)
