"""Locally periodic (RBF x periodic) kernel module
(reference: kernel_matmul/gpytorch/locally_periodic.py:11-140).

The reference passes "spectral" as the native kernel name while stacking four parameters
(locally_periodic.py:33, 130-134); the native kernel that matches those parameters is
"locally_periodic", which is what is used here.
"""
from __future__ import annotations

import multiprocessing.pool

import torch
from torch import Size

from .base import KernelMatmulKernel


class LocallyPeriodicKernelMatmulKernel(KernelMatmulKernel):
    """kernel_value = outputscale * exp(-0.5 (x1 - x2)^2 / lengthscale_rbf^2
    - 2 sin(pi (x1 - x2) / period_length)^2 / lengthscale_periodic)"""

    KERNEL_TYPE = "locally_periodic"
    PARAMETERS = ("lengthscale_rbf", "lengthscale_periodic", "period_length", "outputscale")
    LENGTHSCALES = ("lengthscale_rbf", "lengthscale_periodic")

    def __init__(
        self,
        cutoff: float | None = None,
        epsilon: float | None = None,
        batch_shape: Size = torch.Size(()),
        lengthscale_rbf_constraint=None,
        lengthscale_rbf_prior=None,
        lengthscale_periodic_constraint=None,
        lengthscale_periodic_prior=None,
        outputscale_constraint=None,
        outputscale_prior=None,
        period_length_constraint=None,
        period_length_prior=None,
        compile_pool: multiprocessing.pool.Pool | None = None,
    ):
        super().__init__(self.KERNEL_TYPE, cutoff, epsilon, batch_shape, compile_pool=compile_pool)
        self._register_hyperparameters(
            batch_shape,
            dict(lengthscale_rbf=lengthscale_rbf_constraint,
                 lengthscale_periodic=lengthscale_periodic_constraint,
                 period_length=period_length_constraint, outputscale=outputscale_constraint),
            dict(lengthscale_rbf=lengthscale_rbf_prior,
                 lengthscale_periodic=lengthscale_periodic_prior,
                 period_length=period_length_prior, outputscale=outputscale_prior),
        )
