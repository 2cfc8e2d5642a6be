"""Sparsity patterns: per 128-row block the column interval [start, end) that is kept.

Signatures follow kernel_matmul/ranges.py:39-156 of the reference.  Differences in mechanism:
the builders live in the ahead-of-time library (nothing is compiled at import), and inputs
that already live on the GPU are processed there instead of being copied to the host and back.
"""
from __future__ import annotations

import math

import torch
from torch import Tensor

from kernel_matmul_amd import _BLOCK_SIZE, _native


def _flatten(t: Tensor) -> Tensor:
    if t.dim() == 1:
        return t.unsqueeze(0)
    if t.dim() == 2:
        return t
    return t.reshape(-1, t.shape[-1])


def _ascending(t: Tensor) -> bool:
    return t.shape[-1] < 2 or bool(torch.all(t[..., 1:] >= t[..., :-1]))


def make_ranges(
    cutoff: float | None,
    x1: Tensor,
    x2: Tensor | None = None,
    *,
    block_size: int = _BLOCK_SIZE,
    align: bool = False,
    check_sorted: bool = True,
) -> tuple[Tensor, Tensor]:
    """Compute the sparsity pattern for a cutoff distance.

    Inputs are expected sorted ascending along their last dimension.  Host tensors go through
    the sequential scan of the reference (native/ranges/ranges.cpp:8-101), which returns some
    pattern for unsorted data too; GPU tensors are processed on the GPU by binary searches
    that agree with the scan bit for bit on sorted data only.

    Args:
        cutoff: entries with ``|x1[i] - x2[j]| > cutoff`` may be dropped; ``None`` keeps all.
        x1: sorted inputs of shape ``(batch..., n1)``.
        x2: sorted inputs of shape ``(batch..., n2)``; ``None`` builds the symmetric,
            block-aligned pattern of ``x1`` against itself.
        block_size: rows per block.
        align: restrict start/end to multiples of ``block_size`` (or ``n2``) so that the
            pattern can be transposed exactly.
        check_sorted: verify GPU inputs (one host synchronisation, which the reference's
            device-to-host copy of every input implies as well) and run unsorted ones through the
            host scan, so that the result never depends on the tensors' device.  Callers that
            guarantee sorted input and must not synchronise (stream capture, tight loops) pass
            ``False``: the device builders then run unconditionally.

    Returns:
        ``(start, end)``, int32 tensors of shape ``(batch..., ceil(n1 / block_size))`` on
        ``x1``'s device.
    """
    batch_shape = x1.shape[:-1]
    x1f = _flatten(x1)
    x2f = _flatten(x2) if x2 is not None else None
    rows = int(math.ceil(x1f.shape[1] / block_size))

    if cutoff is None:
        n2 = x2f.shape[1] if x2f is not None else x1f.shape[1]
        start = torch.zeros(x1f.shape[0], rows, dtype=torch.int32, device=x1.device)
        end = torch.full((x1f.shape[0], rows), n2, dtype=torch.int32, device=x1.device)
    else:
        if check_sorted and x1f.is_cuda and not (_ascending(x1f) and (x2f is None or _ascending(x2f))):
            device = x1f.device
            start, end = _native.make_ranges_2d(
                x1f.cpu(), x2f.cpu() if x2f is not None else None, cutoff, block_size, align
            )
            start, end = start.to(device), end.to(device)
        else:
            start, end = _native.make_ranges_2d(x1f, x2f, cutoff, block_size, align)

    return start.reshape(*batch_shape, rows), end.reshape(*batch_shape, rows)


def transpose_ranges(
    start: Tensor, end: Tensor, x1_size: int, x2_size: int, *, block_size: int = _BLOCK_SIZE
) -> tuple[Tensor, Tensor]:
    """Pattern of the transposed matrix; the input pattern must be block aligned.

    Raises:
        ValueError: if some start or end is neither a multiple of ``block_size`` nor ``x2_size``.
    """
    unaligned_start = (start % block_size != 0) & (start != x2_size)
    unaligned_end = (end % block_size != 0) & (end != x2_size)
    if bool(torch.any(unaligned_start | unaligned_end)):
        raise ValueError("Ranges must be block-aligned")

    batch_shape = start.shape[:-1]
    start_t, end_t = _native.transpose_ranges_2d(
        _flatten(start), _flatten(end), x1_size, x2_size, block_size
    )
    return (
        start_t.reshape(*batch_shape, start_t.shape[-1]),
        end_t.reshape(*batch_shape, end_t.shape[-1]),
    )


class RangesCache:
    """Patterns of a fixed ``x = x1 = x2`` memoised by cutoff; index it like a dict."""

    def __init__(self, x: Tensor, align: bool = False):
        self._x = x
        self._align = align
        self._cache: dict[float | None, tuple[Tensor, Tensor]] = {}

    @property
    def x(self) -> Tensor:
        return self._x

    @property
    def align(self) -> bool:
        return self._align

    def __getitem__(self, cutoff: float | None) -> tuple[Tensor, Tensor]:
        if cutoff not in self._cache:
            self._cache[cutoff] = make_ranges(cutoff, self._x, align=self._align)
        return self._cache[cutoff]
