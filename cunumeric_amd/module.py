"""Module-level sort family: ``sort, argsort, msort, sort_complex, partition, argpartition``
and ``searchsorted``, ``unique``.

Same names, arguments, result dtypes / shapes and exceptions as the reference's
"Sorting" section (cunumeric/module.py:6886-7187).
"""
from __future__ import annotations

from typing import Any, Optional, Sequence, Union

import numpy as np
import torch

from .array import convert_to_cunumeric_ndarray, ndarray


def argsort(a: Any, axis: Union[int, None] = -1, kind: str = "quicksort", order=None) -> ndarray:
    """Indices that would sort ``a`` along ``axis`` (``None``: the flattened array);
    int64, same shape as ``a`` (reference: cunumeric/module.py:6886-6929)."""
    a = convert_to_cunumeric_ndarray(a)
    result = ndarray(a.shape, np.int64)
    result._thunk_sort(rhs=a, argsort=True, axis=axis, kind=kind, order=order)
    return result


def msort(a: Any) -> ndarray:
    """Sorted copy along the first axis (reference: cunumeric/module.py:6932-6955)."""
    return sort(a, axis=0)


def unique(ar: Any, return_index: bool = False, return_inverse: bool = False,
           return_counts: bool = False, axis: Optional[int] = None) -> ndarray:
    """The sorted unique elements of ``ar`` (flattened).  As in the reference, the optional
    outputs and ``axis`` are not supported (reference: cunumeric/module.py:6800-6874)."""
    if any((return_index, return_inverse, return_counts, axis)):
        raise NotImplementedError("Keyword arguments for `unique` are not yet supported")
    return convert_to_cunumeric_ndarray(ar).unique()


def searchsorted(a: Any, v: Any, side: str = "left", sorter: Optional[Any] = None):
    """Indices into the sorted 1-D array ``a`` at which the elements of ``v`` would be
    inserted to keep it sorted (reference: cunumeric/module.py:6959-6996)."""
    return convert_to_cunumeric_ndarray(a).searchsorted(v, side, sorter)


def digitize(x: Any, bins: Any, right: bool = False) -> ndarray:
    """Index of the bin every element of ``x`` belongs to: ``searchsorted`` of ``x`` into the
    monotonic 1-D ``bins`` with the side swapped; decreasing bins are searched reversed and the
    result counted from the other end.  Complex ``x`` is a TypeError, bins of more than one
    dimension or not monotonic a ValueError (reference: cunumeric/module.py:9215-9323)."""
    x = convert_to_cunumeric_ndarray(x)
    bins = convert_to_cunumeric_ndarray(bins)
    if x.dtype.kind == "c":
        raise TypeError("x may not be complex")
    if bins.ndim > 1:
        raise ValueError("bins must be one-dimensional")
    b = bins.to_torch().reshape(-1)
    increasing = bool((b[1:] >= b[:-1]).all())
    decreasing = bool((b[1:] <= b[:-1]).all())
    if not increasing and not decreasing:
        raise ValueError("bins must be monotonically increasing or decreasing")
    side = "left" if right else "right"  # backwards because the arguments are swapped
    if increasing:
        return searchsorted(bins, x, side=side)
    flipped = ndarray((b.numel(),), bins.dtype, _buf=b.flip(0).contiguous().view(torch.uint8))
    found = searchsorted(flipped, x, side=side)
    t = found.to_torch() if isinstance(found, ndarray) else None
    if t is None:  # scalar x
        return int(b.numel()) - found
    return ndarray(found.shape, np.int64, _buf=(b.numel() - t).contiguous().reshape(-1).view(torch.uint8))


def sort(a: Any, axis: Union[int, None] = -1, kind: str = "quicksort", order=None) -> ndarray:
    """Sorted copy of ``a`` along ``axis`` (``None``: flattened)
    (reference: cunumeric/module.py:6999-7040)."""
    a = convert_to_cunumeric_ndarray(a)
    result = ndarray(a.shape, a.dtype)
    result._thunk_sort(rhs=a, axis=axis, kind=kind, order=order)
    return result


def sort_complex(a: Any) -> ndarray:
    """Sort along the last axis and return a complex array: integers of at most 16 bits
    promote to complex64, everything else to complex128
    (reference: cunumeric/module.py:7043-7078)."""
    result = sort(a)
    dt = result.dtype
    if dt.kind == "c":
        return result
    narrow_int = dt.kind in "iu" and dt.itemsize <= 2
    return result.astype(np.complex64 if narrow_int else np.complex128, copy=True)


def argpartition(
    a: Any,
    kth: Union[int, Sequence[int]],
    axis: Union[int, None] = -1,
    kind: str = "introselect",
    order=None,
) -> ndarray:
    """Falls back to a full argsort, as the reference does
    (cunumeric/module.py:7084-7137)."""
    a = convert_to_cunumeric_ndarray(a)
    result = ndarray(a.shape, np.int64)
    result._thunk_partition(
        rhs=a, argpartition=True, kth=kth, axis=axis, kind=kind, order=order
    )
    return result


def partition(
    a: Any,
    kth: Union[int, Sequence[int]],
    axis: Union[int, None] = -1,
    kind: str = "introselect",
    order=None,
) -> ndarray:
    """Falls back to a full sort, as the reference does (cunumeric/module.py:7140-7187)."""
    a = convert_to_cunumeric_ndarray(a)
    result = ndarray(a.shape, a.dtype)
    result._thunk_partition(rhs=a, kth=kth, axis=axis, kind=kind, order=order)
    return result
