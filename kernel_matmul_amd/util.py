"""Small helpers shared by the configuration tables and the tests."""
from __future__ import annotations

import itertools
from typing import Any, TypeVar

K = TypeVar("K")
V = TypeVar("V")


def format_dict(d: dict[str, Any]) -> str:
    """``dict(a=1, b=2)`` style rendering (reference: kernel_matmul/util.py:11-13)."""
    return "dict(" + ", ".join(f"{key}={value}" for key, value in d.items()) + ")"


def dict_product(*factors: list[dict[K, V]]) -> list[dict[K, V]]:
    """Cartesian product of lists of dicts, merging one dict per factor.

    Empty factors are skipped; all dicts of one factor must share their keys
    (reference: kernel_matmul/util.py:20-40).
    """
    used = [factor for factor in factors if factor]
    for factor in used:
        keys = set(factor[0])
        for entry in factor[1:]:
            if set(entry) != keys:
                raise ValueError("All dicts in a factor must have the same keys")
    merged = []
    for combination in itertools.product(*used):
        out: dict[K, V] = {}
        for entry in combination:
            out.update(entry)
        merged.append(out)
    return merged
