"""GPyTorch kernel modules that return a KernelMatmulLinearOperator
(reference: kernel_matmul/gpytorch/__init__.py:1-12).  Needs the ``gpytorch`` package."""
from .base import KernelMatmulKernel
from .locally_periodic import LocallyPeriodicKernelMatmulKernel
from .rbf import RBFKernelMatmulKernel
from .spectral import SpectralKernelMatmulKernel
from .sum import SumKernel

__all__ = [
    "KernelMatmulKernel",
    "LocallyPeriodicKernelMatmulKernel",
    "RBFKernelMatmulKernel",
    "SpectralKernelMatmulKernel",
    "SumKernel",
]
