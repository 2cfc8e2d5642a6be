"""LinearOperator over the on-the-fly kernel matrix and the autograd wiring of the native ops.

Mirrors kernel_matmul/linear_operator.py:22-289 of the reference: same constructor, same
batch broadcasting (stride-0 ``expand`` views, no copies), same hooks
(``_matmul``, ``_size``, ``_transpose_nonbatch``, ``to_dense``, ``_expand_batch``, ``to``,
``type``, ``_bilinear_derivative``, ``_get_indices``).

The ``linear_operator`` package is optional.  When it is installed the class derives from
``linear_operator.LinearOperator`` and plugs into GPyTorch's solvers; when it is not, a small
stand-in base supplies ``shape``/``size``/``matmul``/``@``/``transpose``/``diagonal`` so that
the operator remains usable (and testable) on its own.

Two additions over the reference: the backward of ``matmul`` also returns the gradient with
respect to ``rhs`` (``K^T @ grad`` through the same forward kernel on the transposed
pattern), and ``_IndexOperator.backward`` unpacks its saved tensors correctly for batched
operators (the reference slices ``[:8]`` into 7 names, linear_operator.py:71).
"""
from __future__ import annotations

import multiprocessing.pool
from typing import List, Tuple

import torch
from torch import Size, Tensor, dtype

from kernel_matmul_amd import ranges
from kernel_matmul_amd.configurations import (
    BilinearDerivativeConfiguration,
    DenseBwdConfiguration,
    DenseConfiguration,
    IndexBwdConfiguration,
    IndexConfiguration,
    MatmulAutotuneConfiguration,
    MatmulBwdConfiguration,
)
from kernel_matmul_amd.native_function import NativeFunction

try:  # pragma: no cover - depends on the environment
    from linear_operator import LinearOperator
    from linear_operator.utils.generic import _to_helper

    HAVE_LINEAR_OPERATOR = True
except ImportError:
    HAVE_LINEAR_OPERATOR = False

    class LinearOperator:  # type: ignore[no-redef]
        """Minimal stand-in used when the ``linear_operator`` package is absent."""

        def __init__(self, *args, **kwargs):
            self._args = args
            self._kwargs = kwargs

        @property
        def shape(self) -> Size:
            return self._size()

        def size(self, dim: int | None = None):
            return self.shape if dim is None else self.shape[dim]

        def dim(self) -> int:
            return len(self.shape)

        @property
        def batch_shape(self) -> Size:
            return self.shape[:-2]

        @property
        def device(self):
            return self._args[0].device

        @property
        def dtype(self):
            return self._args[0].dtype

        def matmul(self, other: Tensor) -> Tensor:
            if other.dim() == 1:
                return self._matmul(other.unsqueeze(-1)).squeeze(-1)
            return self._matmul(other)

        __matmul__ = matmul

        def transpose(self, dim1: int, dim2: int):
            ndim = self.dim()
            if {dim1 % ndim, dim2 % ndim} != {ndim - 2, ndim - 1}:
                raise NotImplementedError("only the two matrix dimensions can be transposed")
            return self._transpose_nonbatch()

        @property
        def mT(self):
            return self._transpose_nonbatch()

        def expand(self, *sizes):
            if len(sizes) == 1 and not isinstance(sizes[0], int):
                sizes = tuple(sizes[0])
            return self._expand_batch(Size(sizes[:-2]))

        def diagonal(self) -> Tensor:
            if hasattr(self, "_diagonal"):
                return self._diagonal()
            n = min(self.shape[-2], self.shape[-1])
            index = torch.arange(n, device=self.device)
            batch = torch.meshgrid(
                *(torch.arange(s, device=self.device) for s in self.batch_shape), index, indexing="ij"
            )
            return self._get_indices(batch[-1], batch[-1], *batch[:-1])

        def to(self, *args, **kwargs):
            return self

        def type(self, dtype):
            return self

    def _to_helper(*args, **kwargs):
        device = kwargs.get("device")
        dtype_ = kwargs.get("dtype")
        for arg in args:
            if isinstance(arg, torch.dtype):
                dtype_ = arg
            elif isinstance(arg, (str, torch.device)):
                device = torch.device(arg)
        return device, dtype_


class _MatmulOperator(torch.autograd.Function):
    """K @ rhs with gradients for the hyper-parameters (matmul_bwd) and for rhs (K^T @ grad)."""

    @staticmethod
    def forward(ctx, x1, x2, rhs, params, start, end, native_matmul, native_matmul_bwd, symmetric=False,
                transposed_ranges=None):
        ctx.save_for_backward(x1, x2, rhs, params, start, end)
        ctx.native_matmul = native_matmul
        ctx.native_matmul_bwd = native_matmul_bwd
        ctx.symmetric = symmetric
        ctx.transposed_ranges = transposed_ranges  # callable returning (start_t, end_t), or None
        return native_matmul(x1, x2, rhs, params, start, end)

    @staticmethod
    def backward(ctx, grad_output):
        x1, x2, rhs, params, start, end = ctx.saved_tensors
        grad_params = None
        grad_rhs = None
        if ctx.needs_input_grad[3]:
            grad_params = ctx.native_matmul_bwd(x1, x2, rhs, params, start, end, grad_output)
        if ctx.needs_input_grad[2]:
            if ctx.symmetric:
                start_t, end_t = start, end
            else:
                try:
                    if ctx.transposed_ranges is not None:
                        start_t, end_t = ctx.transposed_ranges(start.shape[:-1])
                    else:
                        start_t, end_t = ranges.transpose_ranges(start, end, x1.shape[-1], x2.shape[-1])
                except ValueError as error:
                    raise RuntimeError(
                        "the gradient with respect to rhs needs the transposed sparsity pattern; "
                        "build the ranges with align=True"
                    ) from error
            grad_rhs = ctx.native_matmul(x2, x1, grad_output, params, start_t, end_t)
        return None, None, grad_rhs, grad_params, None, None, None, None, None, None


class _DenseOperator(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, params, start, end, native_dense, native_dense_bwd):
        ctx.save_for_backward(x1, x2, params, start, end)
        ctx.native_dense_bwd = native_dense_bwd
        return native_dense(x1, x2, params, start, end)

    @staticmethod
    def backward(ctx, grad_output):
        x1, x2, params, start, end = ctx.saved_tensors
        grad = ctx.native_dense_bwd(x1, x2, params, start, end, grad_output)
        return None, None, grad, None, None, None, None


class _IndexOperator(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, params, start, end, native_index, native_index_bwd, row_index,
                col_index, *batch_indices):
        ctx.save_for_backward(x1, x2, params, start, end, row_index, col_index, *batch_indices)
        ctx.native_index_bwd = native_index_bwd
        return native_index(x1, x2, params, start, end, batch_indices, row_index, col_index)

    @staticmethod
    def backward(ctx, grad_output):
        x1, x2, params, start, end, row_index, col_index = ctx.saved_tensors[:7]
        batch_indices = ctx.saved_tensors[7:]
        grad = ctx.native_index_bwd(
            x1, x2, params, start, end, batch_indices, row_index, col_index, grad_output
        )
        return (None, None, grad, None, None, None, None, None, None, *[None for _ in batch_indices])


class KernelMatmulLinearOperator(LinearOperator):
    """The (masked) kernel matrix K(x1, x2) of shape (..., M, N), never materialised.

    Args:
        x1: inputs of shape (..., M, 1), sorted along M.
        x2: inputs of shape (..., N, 1), sorted along N.
        params: kernel hyper-parameters of shape (..., P).
        start, end: sparsity pattern of shape (..., ceil(M / 128)), see ``ranges.make_ranges``.
        kernel_type: "rbf", "spectral" or "locally_periodic" (required).
        symmetric: whether K equals its transpose; determined from ``x1 == x2`` if omitted.
        compile_pool: accepted for compatibility; nothing is compiled at run time.
    """

    def __init__(
        self,
        x1: Tensor,
        x2: Tensor,
        params: Tensor,
        start: Tensor,
        end: Tensor,
        kernel_type: str | None = None,
        symmetric: bool | None = None,
        compile_pool: multiprocessing.pool.Pool | None = None,
    ):
        super().__init__(
            x1, x2, params, start, end,
            kernel_type=kernel_type, symmetric=symmetric, compile_pool=compile_pool,
        )
        if kernel_type is None:
            raise ValueError("kernel_type must be specified")
        if x1.dim() < 2 or x2.dim() < 2 or x1.size(-1) != 1 or x2.size(-1) != 1:
            raise ValueError("x1 and x2 must have shapes (..., M, 1) and (..., N, 1), respectively")
        if symmetric is None:
            symmetric = torch.equal(x1, x2)

        batch_shape = torch.broadcast_shapes(
            x1.shape[:-2], x2.shape[:-2], params.shape[:-1], start.shape[:-1], end.shape[:-1]
        )
        self._x1 = x1.expand(*batch_shape, *x1.shape[-2:])
        self._x2 = x2.expand(*batch_shape, *x2.shape[-2:])
        self._params = params.expand(*batch_shape, params.shape[-1])
        self._start = start.expand(*batch_shape, start.shape[-1])
        self._end = end.expand(*batch_shape, end.shape[-1])
        self._kernel_type = kernel_type
        self._batch_shape = batch_shape
        self._symmetric = symmetric
        self._ranges_t = None  # pattern of the transpose, built on first use
        self._diagonal_indices = None  # index tensors of the diagonal, built on first use
        self._native_args = None  # (batch shape, widened constructor tensors) of the last call

        self._native_matmul = NativeFunction(
            "matmul", MatmulAutotuneConfiguration(kernel_type), compile_pool=compile_pool
        )
        self._native_matmul_bwd = NativeFunction("matmul_bwd", MatmulBwdConfiguration(kernel_type))
        self._native_bilinear_derivative = NativeFunction(
            "bilinear_derivative", BilinearDerivativeConfiguration(kernel_type)
        )
        self._native_index = NativeFunction("index", IndexConfiguration(kernel_type))
        self._native_index_bwd = NativeFunction("index_bwd", IndexBwdConfiguration(kernel_type))
        self._native_dense = NativeFunction("dense", DenseConfiguration(kernel_type))
        self._native_dense_bwd = NativeFunction("dense_bwd", DenseBwdConfiguration(kernel_type))

    # -- helpers -------------------------------------------------------------------------
    def _get_args_for_native(self, batch_shape) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
        """The constructor tensors as stride-0 views of ``batch_shape``.  The views of the tensors
        that carry no gradient (coordinates and pattern) are kept for the last shape asked for:
        solvers call with the same one over and over.  ``params`` is widened on every call, so
        the view belongs to the autograd mode of that call (a view made under ``no_grad`` or
        ``inference_mode`` would cut later calls off from the hyper-parameters' gradient)."""
        batch_shape = tuple(batch_shape)

        def widen(t: Tensor, trailing: int) -> Tensor:
            return t.expand(*batch_shape, *t.shape[-trailing:])

        if self._native_args is None or self._native_args[0] != batch_shape:
            fixed = (
                widen(self._x1.detach().squeeze(-1), 1),
                widen(self._x2.detach().squeeze(-1), 1),
                widen(self._start, 1),
                widen(self._end, 1),
            )
            self._native_args = (batch_shape, fixed)
        x1, x2, start, end = self._native_args[1]
        params = self._params if tuple(self._params.shape[:-1]) == batch_shape else widen(self._params, 1)
        return x1, x2, params, start, end

    def _transposed_ranges(self, batch_shape=None) -> tuple[Tensor, Tensor]:
        """Pattern of K^T, computed once per operator (the check that the pattern is block
        aligned and the host pass both synchronise with the device); optionally widened to
        ``batch_shape`` as stride-0 views."""
        if self._ranges_t is None:
            self._ranges_t = ranges.transpose_ranges(
                self._start, self._end, self._x1.size(-2), self._x2.size(-2)
            )
        start_t, end_t = self._ranges_t
        if batch_shape is not None:
            start_t = start_t.expand(*batch_shape, start_t.shape[-1])
            end_t = end_t.expand(*batch_shape, end_t.shape[-1])
        return start_t, end_t

    # -- LinearOperator hooks ------------------------------------------------------------
    def _matmul(self, rhs: Tensor) -> Tensor:
        if rhs.shape[:-2] == self._batch_shape and rhs.size(-2) == self._x2.size(-2):
            batch_shape, rhs_ = self._batch_shape, rhs  # nothing to broadcast
        else:
            expected = Size((*self._batch_shape, self._x2.size(-2), rhs.size(-1)))
            broadcast = torch.broadcast_shapes(expected, rhs.shape)
            batch_shape = broadcast[:-2]
            rhs_ = rhs.expand(*broadcast)
        x1, x2, params, start, end = self._get_args_for_native(batch_shape)
        result = _MatmulOperator.apply(
            x1, x2, rhs_, params, start, end, self._native_matmul, self._native_matmul_bwd,
            self._symmetric, self._transposed_ranges,
        )
        return result.reshape(*batch_shape, *result.shape[-2:])

    def _size(self) -> Size:
        return Size((*self._batch_shape, self._x1.size(-2), self._x2.size(-2)))

    def _transpose_nonbatch(self) -> "KernelMatmulLinearOperator":
        if self._symmetric:
            return self
        start_t, end_t = self._transposed_ranges()
        return KernelMatmulLinearOperator(
            self._x2, self._x1, self._params, start_t, end_t, kernel_type=self._kernel_type
        )

    def to_dense(self) -> Tensor:
        x1, x2, params, start, end = self._get_args_for_native(self._batch_shape)
        return _DenseOperator.apply(
            x1, x2, params, start, end, self._native_dense, self._native_dense_bwd
        )

    def _expand_batch(self, batch_shape: Size | List[int]) -> "KernelMatmulLinearOperator":
        return KernelMatmulLinearOperator(
            self._x1.expand(*batch_shape, *self._x1.shape[-2:]),
            self._x2.expand(*batch_shape, *self._x2.shape[-2:]),
            self._params.expand(*batch_shape, self._params.shape[-1]),
            self._start.expand(*batch_shape, self._start.shape[-1]),
            self._end.expand(*batch_shape, self._end.shape[-1]),
            kernel_type=self._kernel_type,
        )

    def to(self, *args, **kwargs):
        device, dtype_ = _to_helper(*args, **kwargs)
        if (device is not None and device.type != "cuda") or (
            dtype_ is not None and dtype_ != torch.float32
        ):
            raise NotImplementedError("KernelMatmulLinearOperator only supports CUDA and float32")
        return super().to(*args, **kwargs)

    def type(self, dtype: dtype):
        if dtype != torch.float32:
            raise NotImplementedError("KernelMatmulLinearOperator only supports CUDA and float32")
        return super().type(dtype)

    def _bilinear_derivative(self, left_vecs: Tensor, right_vecs: Tensor) -> Tuple[Tensor | None, ...]:
        batch_shape = torch.broadcast_shapes(
            left_vecs.shape[:-2], right_vecs.shape[:-2], self._batch_shape
        )
        left_vecs = left_vecs.expand(*batch_shape, *left_vecs.shape[-2:])
        right_vecs = right_vecs.expand(*batch_shape, *right_vecs.shape[-2:])
        x1, x2, params, start, end = self._get_args_for_native(batch_shape)
        result = self._native_bilinear_derivative(x1, x2, left_vecs, right_vecs, params, start, end)
        grad = result.reshape(*batch_shape, result.shape[-1])
        # one entry per constructor tensor: x1, x2, params, start, end
        return None, None, grad, None, None

    def _diagonal(self) -> Tensor:
        """The diagonal through the index operator, with its index tensors (int32 views that
        repeat one arange per dimension, no copies) built once per operator instead of by the
        base class's ``arange`` / ``meshgrid`` / dtype conversion on every call."""
        if self._diagonal_indices is None:
            n = min(self._x1.shape[-2], self._x2.shape[-2])
            batch_shape = tuple(self._batch_shape)
            device = self._x1.device
            row = torch.arange(n, dtype=torch.int32, device=device).expand(*batch_shape, n)
            batch = []
            for d, size in enumerate(batch_shape):
                view = [1] * (len(batch_shape) + 1)
                view[d] = size
                batch.append(torch.arange(size, dtype=torch.int32, device=device).view(view).expand(*batch_shape, n))
            self._diagonal_indices = (row, tuple(batch))
        row, batch = self._diagonal_indices
        x1, x2, params, start, end = self._get_args_for_native(self._batch_shape)
        return _IndexOperator.apply(
            x1, x2, params, start, end, self._native_index, self._native_index_bwd, row, row, *batch
        )

    def _get_indices(self, row_index: Tensor, col_index: Tensor, *batch_indices: Tensor) -> Tensor:
        x1, x2, params, start, end = self._get_args_for_native(self._batch_shape)
        shape = torch.broadcast_shapes(
            row_index.shape, col_index.shape, *(b.shape for b in batch_indices)
        )

        def prepare(index: Tensor) -> Tensor:
            return index.expand(*shape).to(device=x1.device, dtype=torch.int32)

        return _IndexOperator.apply(
            x1, x2, params, start, end, self._native_index, self._native_index_bwd,
            prepare(row_index), prepare(col_index), *(prepare(b) for b in batch_indices),
        )
