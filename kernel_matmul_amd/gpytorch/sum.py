"""Sum over one batch dimension of a kernel, e.g. the components of a spectral mixture
(reference: kernel_matmul/gpytorch/sum.py:6-30)."""
from __future__ import annotations

from gpytorch.kernels import Kernel
from torch import Size


class SumKernel(Kernel):
    has_lengthscale = False

    def __init__(self, base_kernel: Kernel, dim: int = -1):
        super().__init__()
        self.base_kernel = base_kernel
        self.dim = dim

    def forward(self, x1, x2, diag: bool = False, **params):
        base = self.base_kernel.forward(x1, x2, diag=diag, **params)
        # negative dims count from the batch dimensions, past the 1 (diag) or 2 matrix dims
        dim = self.dim if self.dim >= 0 else self.dim - (1 if diag else 2)
        return base.sum(dim=dim)

    @property
    def batch_shape(self) -> Size:
        shape = list(self.base_kernel.batch_shape)
        del shape[self.dim]
        return Size(shape)
