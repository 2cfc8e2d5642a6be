"""The binding a maintainer of the reference would add (the Python blocks of INTEGRATION.md,
"Option B") is executed as written - only the library's path is filled in - and its operators are
checked against the float64 oracle: what the document shows is what works.

Tolerances as in tests/test_ops_gpu.py: rtol 1e-4 / atol 1e-5 (gradients relative to their scale).
"""
import os
import re

import numpy as np
import pytest
import torch

from kernel_matmul_amd import _native
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle
from tests.conftest import make_params

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RTOL, ATOL = 1e-4, 1e-5


@pytest.fixture(scope="module")
def stub():
    text = open(os.path.join(ROOT, "INTEGRATION.md"), encoding="utf-8").read()
    option_b = text[text.index("## Option B"):text.index("## Conventions of the C ABI")]
    blocks = re.findall(r"```python\n(.*?)```", option_b, re.S)
    assert len(blocks) == 3, "INTEGRATION.md: expected the matmul, gradient/index and ranges blocks"
    source = "\n".join(blocks).replace('"libkernel_matmul_amd.so"', repr(_native.LIB_PATH))
    namespace = {}
    exec(compile(source, "INTEGRATION.md", "exec"), namespace)
    return namespace


def _case(kernel_type, m, n, k, batch, seed):
    g = torch.Generator().manual_seed(seed)
    x1 = torch.sort(torch.rand(*batch, m, generator=g) * 10, dim=-1)[0]
    x2 = torch.sort(torch.rand(*batch, n, generator=g) * 10, dim=-1)[0]
    start, end = make_ranges(2.0, x1, x2)
    rhs = torch.randn(*batch, n, k, generator=g)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)
    return x1, x2, rhs, make_params(kernel_type, batch), start.contiguous(), end.contiguous()


def _np(*tensors):
    return tuple(t.detach().cpu().numpy() for t in tensors)


@pytest.mark.parametrize("kernel_type,define", [("rbf", "KERNEL_RBF"), ("spectral", "KERNEL_SPECTRAL"),
                                                ("locally_periodic", "KERNEL_LOCALLY_PERIODIC")])
def test_operators_of_the_documented_binding(stub, kernel_type, define):
    device = torch.device("cuda:0")
    x1, x2, rhs, params, start, end = _case(kernel_type, 500, 600, 11, (3,), seed=21)
    dev = tuple(t.to(device) for t in (x1, x2, rhs, params, start, end))
    defines = {define: None, "BLOCK_SIZE": 128}

    out = stub["load_native"]("matmul", defines).call(*dev)
    expected = oracle.matmul(kernel_type, *_np(x1, x2, rhs, params, start, end))
    assert np.all(np.abs(out.cpu().double().numpy() - expected) <= ATOL + RTOL * np.abs(expected))

    g = torch.Generator().manual_seed(22)
    out_grad = torch.randn(3, 500, 11, generator=g)
    out_grad = out_grad / torch.linalg.norm(out_grad, dim=(-2, -1), keepdim=True)
    expected_g = oracle.param_grad(kernel_type, *_np(x1, x2, out_grad, rhs, params, start, end))
    tol = ATOL + RTOL * np.maximum(np.abs(expected_g), np.abs(expected_g).max(axis=-1, keepdims=True))
    got = stub["load_native"]("matmul_bwd", defines).call(*dev, out_grad.to(device))
    assert np.all(np.abs(got.cpu().double().numpy() - expected_g) <= tol)
    got = stub["load_native"]("bilinear_derivative", defines).call(
        dev[0], dev[1], out_grad.to(device), dev[2], dev[3], dev[4], dev[5])
    assert np.all(np.abs(got.cpu().double().numpy() - expected_g) <= tol)

    count = (7, 13)
    batch_index = torch.randint(0, 3, count, generator=g, dtype=torch.int32)
    row_index = torch.randint(0, 500, count, generator=g, dtype=torch.int32)
    col_index = torch.randint(0, 600, count, generator=g, dtype=torch.int32)
    got = stub["load_native"]("index", defines).call(
        dev[0], dev[1], dev[3], dev[4], dev[5], (batch_index.to(device),), row_index.to(device),
        col_index.to(device))
    expected_i = oracle.index(kernel_type, *_np(x1, x2, params, start, end), [batch_index.numpy()],
                              row_index.numpy(), col_index.numpy())
    assert np.all(np.abs(got.cpu().double().numpy() - expected_i) <= ATOL + RTOL * np.abs(expected_i))


def test_ranges_of_the_documented_binding(stub):
    g = torch.Generator().manual_seed(23)
    x = torch.sort(torch.rand(2, 1000, generator=g) * 30, dim=-1)[0]
    start, end = stub["_native"].make_ranges_symmetric(x.to("cuda:0"), 2.5, 128)
    expected_start, expected_end = make_ranges(2.5, x)
    assert start.is_cuda and torch.equal(start.cpu(), expected_start) and torch.equal(end.cpu(), expected_end)


def test_usage_example_of_the_readme():
    """The "Use" block of README.md runs as written; the first row block of its product is checked
    against the oracle."""
    text = open(os.path.join(ROOT, "README.md"), encoding="utf-8").read()
    block = re.search(r"## Use.*?```python\n(.*?)```", text, re.S).group(1)
    namespace = {}
    torch.manual_seed(24)
    exec(compile(block, "README.md", "exec"), namespace)
    x, params, start, end, y = (namespace[name] for name in ("x", "params", "start", "end", "y"))
    assert y.shape == (100_000, 16) and bool(torch.isfinite(y).all())
    # y = K @ rhs with an rhs the block does not keep: linearity pins the operator instead
    rhs = torch.randn(100_000, 16, device=x.device)
    product = namespace["K"] @ rhs
    rows = slice(0, 128)
    first, last = int(start[0]), int(end[0])
    expected = oracle.matmul("spectral", x[rows].cpu().numpy(), x[first:last].cpu().numpy(),
                             rhs[first:last].cpu().numpy(), params.cpu().numpy(),
                             np.array([0], dtype=np.int32), np.array([last - first], dtype=np.int32))
    got = product[rows].cpu().double().numpy()
    assert np.all(np.abs(got - expected) <= ATOL + RTOL * np.abs(expected))
