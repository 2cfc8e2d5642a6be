"""Single-component spectral kernel module (reference: kernel_matmul/gpytorch/spectral.py:11-106).
For several components use a batched instance under ``SumKernel``."""
from __future__ import annotations

import multiprocessing.pool

import torch
from torch import Size

from .base import KernelMatmulKernel


class SpectralKernelMatmulKernel(KernelMatmulKernel):
    """kernel_value = outputscale * exp(-0.5 (x1 - x2)^2 / lengthscale^2) * cos(2 pi frequency (x1 - x2))"""

    KERNEL_TYPE = "spectral"
    PARAMETERS = ("lengthscale", "frequency", "outputscale")
    LENGTHSCALES = ("lengthscale",)

    def __init__(
        self,
        cutoff: float | None = None,
        epsilon: float | None = None,
        batch_shape: Size = torch.Size(()),
        lengthscale_constraint=None,
        lengthscale_prior=None,
        outputscale_constraint=None,
        outputscale_prior=None,
        frequency_constraint=None,
        frequency_prior=None,
        compile_pool: multiprocessing.pool.Pool | None = None,
    ):
        super().__init__(self.KERNEL_TYPE, cutoff, epsilon, batch_shape, compile_pool=compile_pool)
        self._register_hyperparameters(
            batch_shape,
            dict(lengthscale=lengthscale_constraint, frequency=frequency_constraint,
                 outputscale=outputscale_constraint),
            dict(lengthscale=lengthscale_prior, frequency=frequency_prior,
                 outputscale=outputscale_prior),
        )
