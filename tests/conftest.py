"""Shared fixtures.  The example shapes, parameter ranges and stride-0 expanded inputs follow
the reference's own fixture (tests/conftest.py:42-160 of Turakar/kernel-matmul); inputs are
generated on the CPU from a per-test seed and moved to the GPU, so the oracle and the device
kernels see identical bits."""
from __future__ import annotations

import os
import random
import sys
import zlib
from dataclasses import dataclass

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "square: use x2 = x1 and the symmetric pattern")
    config.addinivalue_line("markers", "align: build block-aligned ranges")
    config.addinivalue_line("markers", "stable: linspace x, dense pattern, lengthscales x 0.01 (square only)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def seed(request) -> int:
    value = zlib.crc32(request.node.nodeid.encode())
    random.seed(value)
    np.random.seed(value)
    torch.manual_seed(value)
    return value


@dataclass
class ExampleData:
    x1: torch.Tensor
    x2: torch.Tensor
    rhs: torch.Tensor
    params: torch.Tensor
    start: torch.Tensor
    end: torch.Tensor
    kernel_type: str
    cutoff: float | None

    def numpy(self):
        """Materialised (expanded) float/int arrays for the oracle."""
        f = lambda t: t.detach().cpu().numpy()
        return dict(x1=f(self.x1), x2=f(self.x2), rhs=f(self.rhs), params=f(self.params),
                    start=f(self.start), end=f(self.end))


EXAMPLE_SHAPES = [
    dict(m=128, n=128, batch=(), unsqueeze=None, k=1, cutoff=2.0),
    dict(m=600, n=800, batch=(), unsqueeze=None, k=11, cutoff=2.0),
    dict(m=500, n=500, batch=(3,), unsqueeze=None, k=11, cutoff=2.0),
    dict(m=301, n=201, batch=(3,), unsqueeze=0, k=11, cutoff=None),
    dict(m=301, n=199, batch=(2, 3), unsqueeze=1, k=11, cutoff=2.0),
    dict(m=129, n=130, batch=(), unsqueeze=None, k=65, cutoff=2.0),
    # beyond the reference's list: wider rhs, several row blocks, long ranges
    dict(m=1000, n=1100, batch=(2,), unsqueeze=None, k=32, cutoff=3.0),
    dict(m=257, n=300, batch=(), unsqueeze=None, k=16, cutoff=1.0),
]
KERNEL_TYPES = ["rbf", "spectral", "locally_periodic"]


def make_params(kernel_type: str, batch, lengthscale_factor: float = 1.0) -> torch.Tensor:
    r = lambda: torch.rand(batch)
    if kernel_type == "rbf":
        cols = [(1 + r()) * lengthscale_factor, 1 + r()]
    elif kernel_type == "spectral":
        cols = [(1 + r()) * lengthscale_factor, 0.5 + r() * 0.5, 1 + r()]
    elif kernel_type == "locally_periodic":
        cols = [(1 + r()) * lengthscale_factor, 1 + r() * lengthscale_factor, 1 + r(), 1 + r()]
    else:
        raise ValueError(kernel_type)
    return torch.stack(cols, dim=-1).float()


def build_example(shape: dict, kernel_type: str, device, square=False, align=False,
                  stable=False) -> ExampleData:
    """``stable`` is the regime of the reference's square LinearOperator suite
    (tests/conftest.py:67-91, 114 there): evenly spaced x, no cutoff (every row block covers all
    columns) and lengthscales of 0.01 ... 0.02, so that almost every entry of K underflows."""
    from kernel_matmul_amd.ranges import make_ranges

    if stable and not square:
        pytest.skip("Stable test only implemented for square matrices")
    m = shape["m"]
    n = m if square else shape["n"]
    batch, unsqueeze, k, cutoff = shape["batch"], shape["unsqueeze"], shape["k"], shape["cutoff"]
    if stable:
        cutoff = None
    squeeze_batch = batch if unsqueeze is None else (*batch[:unsqueeze], *batch[unsqueeze + 1:])

    if stable:
        x1 = torch.linspace(0, 10, m).expand(*squeeze_batch, m)
    else:
        x1 = torch.sort(torch.rand(*squeeze_batch, m) * 10, dim=-1)[0]
    x2 = x1 if square else torch.sort(torch.rand(*squeeze_batch, n) * 10, dim=-1)[0]
    if square:
        start, end = make_ranges(cutoff, x1, align=align)
    else:
        start, end = make_ranges(cutoff, x1, x2, align=align)
    rhs = torch.randn(*squeeze_batch, n, k)
    rhs = rhs / torch.linalg.norm(rhs, dim=-2, keepdim=True)
    params = make_params(kernel_type, batch, 0.01 if stable else 1.0)

    x1, x2, rhs, start, end, params = (t.to(device) for t in (x1, x2, rhs, start, end, params))
    if unsqueeze is not None:
        # stride-0 expanded views, the normal case when called from the LinearOperator
        x1 = x1.unsqueeze(unsqueeze).expand(*batch, m)
        x2 = x2.unsqueeze(unsqueeze).expand(*batch, n)
        start = start.unsqueeze(unsqueeze).expand(*batch, -1)
        end = end.unsqueeze(unsqueeze).expand(*batch, -1)
        rhs = rhs.unsqueeze(unsqueeze).expand(*batch, n, k)
    return ExampleData(x1, x2, rhs, params, start, end, kernel_type, cutoff)


@pytest.fixture(
    params=[
        pytest.param((i, kt), id=f"example{i}-{kt}")
        for i in range(len(EXAMPLE_SHAPES))
        for kt in KERNEL_TYPES
    ]
)
def example_data(request) -> ExampleData:
    index, kernel_type = request.param
    square = request.node.get_closest_marker("square") is not None
    align = request.node.get_closest_marker("align") is not None
    stable = request.node.get_closest_marker("stable") is not None
    device = torch.device("cuda:0")
    return build_example(EXAMPLE_SHAPES[index], kernel_type, device, square=square, align=align,
                         stable=stable)
