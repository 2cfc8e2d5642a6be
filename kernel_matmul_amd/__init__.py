"""MI355X-native KernelMatmul: banded K(x1, x2) @ rhs with the kernel matrix evaluated on the
fly by hand-written gfx950 kernels behind a C ABI (see include/kernel_matmul_amd.h).

The Python surface mirrors Turakar/kernel-matmul (``native_function``, ``configurations``,
``compile``, ``ranges``, ``linear_operator``, ``gpytorch``) so code written against that
package runs unchanged.
"""

_BLOCK_SIZE = 128
"""Rows per block of the sparsity pattern; fixed by the device kernels
(reference: kernel_matmul/__init__.py:1)."""

__version__ = "0.1.0"
