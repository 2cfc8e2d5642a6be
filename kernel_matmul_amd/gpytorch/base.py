"""Base class of the GPyTorch kernels (reference: kernel_matmul/gpytorch/base.py:16-84).

A kernel holds its hyper-parameters as constrained ``raw_*`` parameters, stacks them in the
order the native operators expect, builds the block-aligned sparsity pattern for the current
cutoff and hands everything to ``KernelMatmulLinearOperator``.  Subclasses only list their
parameter names (``PARAMETERS``, in native order) and say which of them are lengthscales.
"""
from __future__ import annotations

import abc
import math
import multiprocessing.pool

import torch
from gpytorch.constraints import GreaterThan
from gpytorch.kernels import Kernel
from torch import Size, Tensor, nn

from kernel_matmul_amd.linear_operator import KernelMatmulLinearOperator
from kernel_matmul_amd.ranges import make_ranges


def _parameter_property(name: str) -> property:
    raw = f"raw_{name}"

    def getter(self) -> Tensor:
        return getattr(self, f"{raw}_constraint").transform(getattr(self, raw))

    def setter(self, value) -> None:
        value = torch.as_tensor(value).expand(getattr(self, raw).shape)
        self.initialize(**{raw: getattr(self, f"{raw}_constraint").inverse_transform(value)})

    return property(getter, setter)


class KernelMatmulKernel(Kernel, abc.ABC):
    """Base class for KernelMatmul-based GPyTorch kernels."""

    has_lengthscale = False
    #: native kernel name
    KERNEL_TYPE: str = ""
    #: hyper-parameter names in the order of the native ``params`` tensor
    PARAMETERS: tuple[str, ...] = ()
    #: parameters that count as lengthscales for the epsilon-based cutoff
    LENGTHSCALES: tuple[str, ...] = ()

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        for name in cls.PARAMETERS:
            setattr(cls, name, _parameter_property(name))

    def __init__(
        self,
        kernel_type: str,
        cutoff: float | None,
        epsilon: float | None,
        batch_shape: Size,
        compile_pool: multiprocessing.pool.Pool | None = None,
    ):
        super().__init__(batch_shape=batch_shape)
        if cutoff is not None and epsilon is not None:
            raise ValueError("Cannot have both a fixed cutoff and an epsilon for dynamic cutoff!")
        self._kernel_type = kernel_type
        self._cutoff = cutoff
        self._epsilon = epsilon
        self._compile_pool = compile_pool

    def _register_hyperparameters(self, batch_shape: Size, constraints: dict, priors: dict) -> None:
        """Create ``raw_<name>`` parameters with constraints (default > 1e-6) and optional priors."""
        for name in self.PARAMETERS:
            raw = f"raw_{name}"
            self.register_parameter(raw, nn.Parameter(torch.zeros(batch_shape)))
            constraint = constraints.get(name)
            self.register_constraint(raw, GreaterThan(1e-6) if constraint is None else constraint)
            prior = priors.get(name)
            if prior is not None:
                self.register_prior(
                    f"{name}_prior",
                    prior,
                    lambda module, name=name: getattr(module, name),
                    lambda module, value, name=name: module.initialize(**{name: value}),
                )

    def _get_params(self) -> Tensor:
        return torch.stack([getattr(self, name) for name in self.PARAMETERS], dim=-1)

    def _get_largest_lengthscale(self) -> float:
        return max(getattr(self, name).max().item() for name in self.LENGTHSCALES)

    def _current_cutoff(self) -> float | None:
        if self._epsilon is not None:
            # distance at which a unit Gaussian profile has dropped to epsilon tail mass
            quantile = math.sqrt(2) * torch.special.erfinv(torch.tensor(1 - self._epsilon)).item()
            return quantile * self._get_largest_lengthscale()
        return self._cutoff

    def forward(self, x1: Tensor, x2: Tensor, diag: bool = False, last_dim_is_batch: bool = False,
                **params) -> KernelMatmulLinearOperator | Tensor:
        if last_dim_is_batch:
            raise NotImplementedError("last_dim_is_batch not supported for KernelMatmulKernel")
        symmetric = torch.equal(x1, x2)
        cutoff = self._current_cutoff()
        if symmetric:
            start, end = make_ranges(cutoff, x1.squeeze(-1), align=True)
        else:
            start, end = make_ranges(cutoff, x1.squeeze(-1), x2.squeeze(-1), align=True)
        operator = KernelMatmulLinearOperator(
            x1, x2, self._get_params(), start, end,
            kernel_type=self._kernel_type, symmetric=symmetric, compile_pool=self._compile_pool,
        )
        return operator.diagonal() if diag else operator
