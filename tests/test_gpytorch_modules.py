"""GPyTorch kernel modules (reference: kernel_matmul/gpytorch/*.py).  GPyTorch itself is not
installed in the build environment, so the module logic (parameter order, constraints,
cutoff from epsilon, pattern construction) is exercised against a minimal stand-in of the
three gpytorch names it imports; with the real package present the stand-in is not used."""
import importlib
import math
import sys
import types

import pytest
import torch
from torch import nn


def _install_gpytorch_stub(monkeypatch):
    class GreaterThan:
        def __init__(self, lower):
            self.lower = lower

        def transform(self, raw):
            return torch.nn.functional.softplus(raw) + self.lower

        def inverse_transform(self, value):
            return torch.log(torch.expm1(value - self.lower))

    class Kernel(nn.Module):
        has_lengthscale = False

        def __init__(self, batch_shape=torch.Size(())):
            super().__init__()
            self._batch_shape = batch_shape
            self.priors = {}

        @property
        def batch_shape(self):
            return self._batch_shape

        def register_constraint(self, name, constraint):
            setattr(self, f"{name}_constraint", constraint)

        def register_prior(self, name, prior, closure, setting_closure):
            self.priors[name] = (prior, closure, setting_closure)

        def initialize(self, **kwargs):
            for name, value in kwargs.items():
                if hasattr(type(self), name) and isinstance(getattr(type(self), name), property):
                    setattr(self, name, value)
                else:
                    getattr(self, name).data.copy_(torch.as_tensor(value).expand(getattr(self, name).shape))
            return self

    gpytorch = types.ModuleType("gpytorch")
    kernels = types.ModuleType("gpytorch.kernels")
    constraints = types.ModuleType("gpytorch.constraints")
    kernels.Kernel = Kernel
    constraints.GreaterThan = GreaterThan
    gpytorch.kernels, gpytorch.constraints = kernels, constraints
    for name, module in (("gpytorch", gpytorch), ("gpytorch.kernels", kernels),
                         ("gpytorch.constraints", constraints)):
        monkeypatch.setitem(sys.modules, name, module)
    for name in [m for m in sys.modules if m.startswith("kernel_matmul_amd.gpytorch")]:
        monkeypatch.delitem(sys.modules, name)


@pytest.fixture
def km_gpytorch(monkeypatch):
    try:
        import gpytorch  # noqa: F401
    except ImportError:
        _install_gpytorch_stub(monkeypatch)
    return importlib.import_module("kernel_matmul_amd.gpytorch")


def test_parameter_order_and_properties(km_gpytorch):
    k = km_gpytorch.SpectralKernelMatmulKernel(cutoff=3.0, batch_shape=torch.Size((2,)))
    assert [n for n, _ in k.named_parameters()] == ["raw_lengthscale", "raw_frequency", "raw_outputscale"]
    k.lengthscale = torch.tensor([0.5, 2.0])
    k.frequency = torch.tensor(0.25)
    k.outputscale = torch.tensor([1.5, 0.75])
    params = k._get_params()
    assert params.shape == (2, 3)
    assert torch.allclose(params, torch.tensor([[0.5, 0.25, 1.5], [2.0, 0.25, 0.75]]), atol=1e-6)
    assert abs(k._get_largest_lengthscale() - 2.0) < 1e-6

    lp = km_gpytorch.LocallyPeriodicKernelMatmulKernel(cutoff=1.0)
    assert lp._kernel_type == "locally_periodic"
    assert lp.PARAMETERS == ("lengthscale_rbf", "lengthscale_periodic", "period_length", "outputscale")
    assert lp._get_params().shape == (4,)
    rbf = km_gpytorch.RBFKernelMatmulKernel(epsilon=1e-4)
    assert rbf._get_params().shape == (2,)


def test_cutoff_rules(km_gpytorch):
    with pytest.raises(ValueError, match="Cannot have both a fixed cutoff and an epsilon"):
        km_gpytorch.RBFKernelMatmulKernel(cutoff=1.0, epsilon=1e-3)
    k = km_gpytorch.RBFKernelMatmulKernel(epsilon=1e-3)
    k.lengthscale = torch.tensor(2.0)
    expected = math.sqrt(2) * torch.special.erfinv(torch.tensor(1 - 1e-3)).item() * 2.0
    assert abs(k._current_cutoff() - expected) < 1e-5
    assert km_gpytorch.RBFKernelMatmulKernel()._current_cutoff() is None


def test_forward_builds_aligned_operator(km_gpytorch):
    from kernel_matmul_amd.linear_operator import KernelMatmulLinearOperator

    k = km_gpytorch.SpectralKernelMatmulKernel(cutoff=1.0, batch_shape=torch.Size((3,)))
    x = torch.sort(torch.rand(400, 1) * 20, dim=0)[0]
    op = k.forward(x, x)
    assert isinstance(op, KernelMatmulLinearOperator)
    assert op.shape == (3, 400, 400) and op._symmetric and op._kernel_type == "spectral"
    assert torch.all((op._start % 128 == 0) | (op._start == 400))
    x2 = torch.sort(torch.rand(300, 1) * 20, dim=0)[0]
    op2 = k.forward(x, x2)
    assert op2.shape == (3, 400, 300) and not op2._symmetric
    with pytest.raises(NotImplementedError):
        k.forward(x, x, last_dim_is_batch=True)

    total = km_gpytorch.SumKernel(k)
    assert total.batch_shape == torch.Size(())
