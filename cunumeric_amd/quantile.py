"""``quantile`` / ``percentile`` / ``nanquantile`` / ``nanpercentile``: the callers of the sort
path in the reference's statistics section (cunumeric/module.py:8339-8531 ``quantile``,
8534-8644 ``percentile``, which sort the array along the reduction axis with ``sort`` /
``ndarray.sort`` at :8472-8476 and then read the two order statistics around each quantile,
``quantile_impl`` :8248-8336; :8757-8962 ``nanquantile`` and :8965-9065 ``nanpercentile``, which
count the non-NaN elements of every slice, sort with the NaNs moved behind everything else
(:8901-8903) and read the order statistics of each slice's own length, ``nanquantile_impl``
:8647-8754).

Same arguments, result shapes / dtypes and exceptions.  The order statistics come from the
GPU sort of this package; for a few quantiles over a flat array or long rows they come from the
selection behind ``partition`` instead, which moves no row (the reference's own comment at
:8462-8467 names partitioning as the cheaper way it does not take).  Picking the two neighbours out of the sorted array
and blending them is elementwise arithmetic, which is not part of the sort path: it runs
through torch on the device.  NumPy defines the 13 methods (numpy.quantile); the position of
a quantile in the sorted sample and its blending weight follow NumPy's definitions, so
results match numpy.quantile to rounding.
"""
from __future__ import annotations

import math
from typing import Any, Iterable, Optional, Sequence, Union

import numpy as np
import torch

from .array import _TORCH_TO_NUMPY, convert_to_cunumeric_ndarray, ndarray

# Hyndman & Fan's plotting-position constants (alpha, beta) of the continuous methods: the
# quantile q of n sorted samples sits at position n*q + alpha + q*(1 - alpha - beta) - 1.
_CONTINUOUS = {
    "interpolated_inverted_cdf": (0.0, 1.0),
    "hazen": (0.5, 0.5),
    "weibull": (0.0, 0.0),
    "median_unbiased": (1.0 / 3.0, 1.0 / 3.0),
    "normal_unbiased": (3.0 / 8.0, 3.0 / 8.0),
}
# methods that return one of the samples: the result keeps the input's dtype
_SAMPLE_METHODS = ("inverted_cdf", "closest_observation", "lower", "higher", "nearest")
METHODS = ("inverted_cdf", "averaged_inverted_cdf", "closest_observation", "interpolated_inverted_cdf",
           "hazen", "weibull", "linear", "median_unbiased", "normal_unbiased", "lower", "higher",
           "midpoint", "nearest")


def _round_half_even(x: float) -> int:
    f = math.floor(x)
    d = x - f
    if d > 0.5 or (d == 0.5 and f % 2 == 1):
        return int(f) + 1
    return int(f)


def _position(method: str, q: float, n: int) -> tuple[int, int, float]:
    """Where quantile ``q`` of ``n`` sorted samples lies: indices (lo, hi) of the two samples
    and the weight g of the upper one; the quantile is lerp(x[lo], x[hi], g)."""
    last = n - 1

    def clipped(v: float, weight) -> tuple[int, int, float]:
        # beyond the ends the quantile is the extreme sample
        if v >= last:
            return last, last, 0.0
        if v < 0:
            return 0, 0, 0.0
        lo = math.floor(v)
        return int(lo), int(lo) + 1, weight(v - lo, v)

    if method in _CONTINUOUS or method == "linear":
        if method == "linear":
            v = last * q  # same position as alpha = beta = 1, with less rounding
        else:
            alpha, beta = _CONTINUOUS[method]
            v = n * q + (alpha + q * (1.0 - alpha - beta)) - 1.0
        return clipped(v, lambda frac, _: frac)
    if method == "averaged_inverted_cdf":
        return clipped(n * q - 1.0, lambda frac, _: 0.5 if frac == 0 else 1.0)
    if method == "midpoint":
        v = 0.5 * (math.floor(last * q) + math.ceil(last * q))
        return clipped(v, lambda frac, vv: 0.0 if vv % 1 == 0 else 0.5)
    # the remaining methods name one sample
    if method == "inverted_cdf":
        v = n * q - 1.0
        lo = math.floor(v)
        i = lo if v == lo else lo + 1
    elif method == "closest_observation":
        v = n * q - 1.5
        lo = math.floor(v)
        # on a tie take the order statistic with the even 1-based rank
        i = lo if (v == lo and lo % 2 == 1) else lo + 1
    elif method == "lower":
        i = math.floor(last * q)
    elif method == "higher":
        i = math.ceil(last * q)
    elif method == "nearest":
        i = _round_half_even(last * q)
    else:
        raise ValueError(f"{method!r} is not a valid method. Use one of: {', '.join(METHODS)}")
    i = min(max(int(i), 0), last)
    return i, i, 0.0


def _torch_dtype(dtype) -> torch.dtype:
    for t, n in _TORCH_TO_NUMPY.items():
        if np.dtype(n) == np.dtype(dtype):
            return t
    raise TypeError(dtype)


def _from_torch(t: torch.Tensor, dtype) -> ndarray:
    t = t.contiguous()
    return ndarray(tuple(t.shape), dtype, _buf=t.reshape(-1).view(torch.uint8))


def _select_rows(a: ndarray, k: int, want_next: bool):
    """The elements at sorted positions k (and k + 1) of every row of ``a`` and the rows' last
    element in sort order, by the library's selection (no row is moved); ``None`` where the
    library does not serve the case."""
    from . import _lib
    from .config import to_core_dtype
    from .runtime import runtime

    lib = _lib.load()
    code = to_core_dtype(a.dtype)
    n = a.shape[-1]
    need = lib.misort_select_scratch_bytes(code, a.size, n, k)
    if not need:
        return None
    rows = a.size // n
    scratch = runtime.alloc_bytes(need)
    outs = [ndarray((rows,), a.dtype) for _ in range(3 if want_next else 2)]
    kth, top = outs[0], outs[-1]
    _lib.check(lib.misort_select(code, a._ptr(), a.size, n, k, kth._ptr(), outs[1]._ptr() if want_next else None,
                                 top._ptr(), scratch.data_ptr(), need, runtime.stream_handle()))
    shape = tuple(a.shape[:-1])
    return [o.to_torch().reshape(shape) for o in outs]


def _order_statistics(a: ndarray, wanted: Sequence[int], overwrite_input: bool, exact_bits: bool = False):
    """``a`` has the reduction axis last: the samples at the sorted positions ``wanted`` of
    every row, as tensors of the row shape, and (or None) which rows hold a NaN.  A few
    positions on long rows are found by selection, one call per position or adjacent pair: two
    reads of the rows each instead of a sort (which moves them once or twice per key byte), and
    the rows' largest element, which comes with it, tells the NaNs.  Anything else sorts the
    rows.  The selection hands floating-point samples back as their keys keep them (a zero as
    +0): ``exact_bits`` (the methods that return a sample itself) keeps floating-point rows on
    the sort, so that the sample carries the bit pattern the sorted row has at that position
    whatever the row length.  ``overwrite_input`` permits the sort to run in place; the
    selection leaves the input as it is, which the permission covers."""
    from .module import sort

    n = a.shape[-1]
    wanted = sorted(set(wanted))
    pairs: list[tuple[int, bool]] = []  # (position, the next one is wanted too)
    for k in wanted:
        if pairs and pairs[-1][0] + 1 == k and not pairs[-1][1]:
            pairs[-1] = (k - 1, True)
        elif not (pairs and pairs[-1][1] and pairs[-1][0] + 1 == k):
            pairs.append((k, False))
    # a selection costs about two reads of the rows, a sort two (one read, one write) per key byte
    if (0 < len(pairs) <= a.dtype.itemsize // 2 + 1 and n >= (1 << 16) and a.dtype.itemsize >= 4 and
            a.dtype.kind in "fiu" and a.size and not (exact_bits and a.dtype.kind == "f")):
        out: dict[int, torch.Tensor] = {}
        top = None
        for k, with_next in pairs:
            found = _select_rows(a, k, with_next)
            if found is None:
                break
            out[k] = found[0]
            if with_next:
                out[k + 1] = found[1]
            top = found[-1]
        else:
            return out, (torch.isnan(top) if a.dtype.kind == "f" else None)
    if overwrite_input:
        a.sort(axis=-1)
        s = a
    else:
        s = sort(a, axis=-1)
    t = s.to_torch()
    # (NaNs sort last)
    has_nan = torch.isnan(t[..., -1]) if a.dtype.kind == "f" and n else None
    return {k: t[..., k] for k in wanted}, has_nan


def _reduction_rows(a: ndarray, axis):
    """``a`` with the reduction axes moved last and merged into one: (rows, axes, shape of the
    kept axes, original shape, whether that needed a copy)."""
    original_shape = a.shape
    nd = a.ndim
    if axis is None:
        axes = tuple(range(nd))
    elif isinstance(axis, Iterable):
        axes = tuple(int(x) for x in axis)
    else:
        axes = (int(axis),)
    norm = []
    for x in axes:
        if not -nd <= x < nd:
            raise ValueError(f"axis {x} is out of bounds for an array of dimension {nd}")
        norm.append(x % nd if nd else 0)
    if len(set(norm)) != len(norm):
        raise ValueError("repeated axis")
    axes = tuple(norm)
    kept = tuple(k for k in range(nd) if k not in axes)
    n = 1
    for k in axes:
        n *= original_shape[k]
    if nd == 0:
        n = 1
    if n == 0:
        raise ValueError("cannot take a quantile of an empty sample")
    kept_shape = tuple(original_shape[k] for k in kept)
    if nd and (kept + axes) != tuple(range(nd)):
        # a dense copy with the reduced axes moved behind the others (never sorted in place)
        moved = a.to_torch().permute(*kept, *axes).contiguous()
        return _from_torch(moved.reshape(*kept_shape, n), a.dtype), axes, kept_shape, original_shape, True
    return a.reshape((*kept_shape, n)), axes, kept_shape, original_shape, False


def quantile(a: Any, q: Any, axis: Union[None, int, Iterable[int]] = None, out: Optional[ndarray] = None,
             overwrite_input: bool = False, method: str = "linear", keepdims: bool = False) -> ndarray:
    """The q-th quantile(s) of ``a`` along ``axis`` (``None``: of the flattened array; several
    axes: of their product).  Result shape: ``q.shape`` followed by the shape of ``a`` without
    the reduced axes (kept with extent 1 under ``keepdims``); dtype: the input's for the methods
    that return a sample, float64 otherwise; complex input is a TypeError, a wrongly shaped
    ``out`` a ValueError (reference: cunumeric/module.py:8339-8531)."""
    if method not in METHODS:
        raise ValueError(f"{method!r} is not a valid method. Use one of: {', '.join(METHODS)}")
    a = convert_to_cunumeric_ndarray(a)
    if a.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    q_arr = np.asarray(q, dtype=np.float64)
    if q_arr.size and not (np.all(q_arr >= 0) and np.all(q_arr <= 1)):
        raise ValueError("Quantiles must be in the range [0, 1]")
    rows, axes, kept_shape, original_shape, moved = _reduction_rows(a, axis)
    nd = a.ndim
    n = rows.shape[-1]
    if moved or (len(axes) > 1 and axis is not None):
        overwrite_input = False  # as the reference: only a single axis is sorted in place

    # ---- the samples around every quantile ---------------------------------------------
    places = [_position(method, float(qv), n) for qv in q_arr.reshape(-1)]
    wanted = [p[0] for p in places] + [p[1] for p in places]
    stats, has_nan = _order_statistics(rows, wanted, overwrite_input, exact_bits=method in _SAMPLE_METHODS)
    to_dtype = a.dtype if method in _SAMPLE_METHODS else np.dtype(np.float64)
    tdt = _torch_dtype(to_dtype)
    results = []
    for lo, hi, g in places:
        if lo == hi or g == 0.0:
            r = stats[lo].to(tdt)
        else:
            x, y = stats[lo].to(tdt), stats[hi].to(tdt)
            d = y - x
            # the upper sample anchors the blend from the middle on, as in NumPy
            r = x + d * g if g < 0.5 else y - d * (1.0 - g)
        results.append(r)
    res = torch.stack(results, dim=0) if results else torch.empty((0, *kept_shape), dtype=tdt,
                                                                  device=rows.to_torch().device)
    if has_nan is not None and results:
        # a sample with a NaN has no quantiles: its last element in sort order tells
        nan = torch.tensor(float("nan"), dtype=tdt, device=res.device)
        res = torch.where(has_nan.unsqueeze(0), nan, res)
    if keepdims:
        remaining = tuple(1 if k in axes else original_shape[k] for k in range(nd))
    else:
        remaining = kept_shape
    shape = (*q_arr.shape, *remaining)
    res = res.reshape(shape)
    if out is not None:
        if tuple(out.shape) != shape:
            raise ValueError("wrong shape on output array")
        out.to_torch().copy_(res.to(_torch_dtype(out.dtype)))
        return out
    return _from_torch(res, to_dtype)


def percentile(a: Any, q: Any, axis: Union[None, int, Iterable[int]] = None, out: Optional[ndarray] = None,
               overwrite_input: bool = False, method: str = "linear", keepdims: bool = False) -> ndarray:
    """The q-th percentile(s): ``quantile`` with ``q / 100``
    (reference: cunumeric/module.py:8534-8644)."""
    q_arr = np.true_divide(np.asarray(q, dtype=np.float64), 100.0)
    if q_arr.size and not (np.all(q_arr >= 0) and np.all(q_arr <= 1)):
        raise ValueError("Percentiles must be in the range [0, 100]")
    return quantile(a, q_arr, axis=axis, out=out, overwrite_input=overwrite_input, method=method,
                    keepdims=keepdims)


def _position_rows(method: str, q: float, n: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``_position`` for samples of different sizes at once: ``n`` holds the size of every
    sample (int64, >= 1); returns int64 lo, hi and float64 g of the same shape."""
    nf = n.to(torch.float64)
    last = nf - 1.0

    def clipped(v, weight):
        lo = torch.floor(v)
        g = weight(v - lo, v)
        over, under = v >= last, v < 0
        lo_c = torch.where(over, last, torch.where(under, torch.zeros_like(v), lo))
        hi_c = torch.where(over | under, lo_c, lo + 1.0)
        g_c = torch.where(over | under, torch.zeros_like(v), g)
        return lo_c.to(torch.int64), hi_c.to(torch.int64), g_c

    if method in _CONTINUOUS or method == "linear":
        if method == "linear":
            v = last * q
        else:
            alpha, beta = _CONTINUOUS[method]
            v = nf * q + (alpha + q * (1.0 - alpha - beta)) - 1.0
        return clipped(v, lambda frac, _: frac)
    if method == "averaged_inverted_cdf":
        return clipped(nf * q - 1.0, lambda frac, _: torch.where(frac == 0, 0.5, 1.0).to(torch.float64))
    if method == "midpoint":
        v = 0.5 * (torch.floor(last * q) + torch.ceil(last * q))
        return clipped(v, lambda frac, _: torch.where(frac == 0, 0.0, 0.5).to(torch.float64))
    if method == "inverted_cdf":
        v = nf * q - 1.0
        lo = torch.floor(v)
        i = torch.where(v == lo, lo, lo + 1.0)
    elif method == "closest_observation":
        v = nf * q - 1.5
        lo = torch.floor(v)
        odd = torch.remainder(lo, 2.0) == 1.0
        i = torch.where((v == lo) & odd, lo, lo + 1.0)
    elif method == "lower":
        i = torch.floor(last * q)
    elif method == "higher":
        i = torch.ceil(last * q)
    elif method == "nearest":
        i = torch.round(last * q)  # half to even
    else:
        raise ValueError(f"{method!r} is not a valid method. Use one of: {', '.join(METHODS)}")
    i = torch.minimum(torch.clamp(i, min=0.0), last).to(torch.int64)
    return i, i, torch.zeros_like(nf)


def nanquantile(a: Any, q: Any, axis: Union[None, int, Iterable[int]] = None, out: Optional[ndarray] = None,
                overwrite_input: bool = False, method: str = "linear", keepdims: bool = False) -> ndarray:
    """The q-th quantile(s) of ``a`` along ``axis``, ignoring NaNs: every slice is its non-NaN
    elements (the sort of this package puts NaNs last, so they are the tail of the sorted
    slice); a slice of NaNs only gives NaN.  Shapes, dtypes and exceptions as ``quantile``
    (reference: cunumeric/module.py:8757-8962, 8647-8754)."""
    from .module import sort

    if method not in METHODS:
        raise ValueError(f"{method!r} is not a valid method. Use one of: {', '.join(METHODS)}")
    a = convert_to_cunumeric_ndarray(a)
    if a.dtype.kind == "c":
        raise TypeError("input array cannot be of complex type")
    q_arr = np.asarray(q, dtype=np.float64)
    if q_arr.size and not (np.all(q_arr >= 0) and np.all(q_arr <= 1)):
        raise ValueError("Quantiles must be in the range [0, 1]")
    rows, axes, kept_shape, original_shape, _ = _reduction_rows(a, axis)
    nd = a.ndim
    t = sort(rows, axis=-1).to_torch()
    if a.dtype.kind == "f":
        count = (~torch.isnan(t)).sum(dim=-1)
    else:
        count = torch.full(kept_shape, t.shape[-1], dtype=torch.int64, device=t.device)
    empty = count == 0
    n = torch.clamp(count, min=1)
    to_dtype = a.dtype if method in _SAMPLE_METHODS else np.dtype(np.float64)
    tdt = _torch_dtype(to_dtype)
    results = []
    for qv in q_arr.reshape(-1):
        lo, hi, g = _position_rows(method, float(qv), n)
        x = t.gather(-1, lo.unsqueeze(-1)).squeeze(-1).to(tdt)
        if method in _SAMPLE_METHODS:
            r = x
        else:
            y = t.gather(-1, hi.unsqueeze(-1)).squeeze(-1).to(tdt)
            d = y - x
            # the upper sample anchors the blend from the middle on, as in NumPy
            r = torch.where(g == 0, x, torch.where(g < 0.5, x + d * g, y - d * (1.0 - g)))
        if a.dtype.kind == "f":
            r = torch.where(empty, torch.tensor(float("nan"), dtype=tdt, device=r.device), r)
        results.append(r)
    res = torch.stack(results, dim=0) if results else torch.empty((0, *kept_shape), dtype=tdt, device=t.device)
    if keepdims:
        remaining = tuple(1 if k in axes else original_shape[k] for k in range(nd))
    else:
        remaining = kept_shape
    shape = (*q_arr.shape, *remaining)
    res = res.reshape(shape)
    if out is not None:
        if tuple(out.shape) != shape:
            raise ValueError("wrong shape on output array")
        out.to_torch().copy_(res.to(_torch_dtype(out.dtype)))
        return out
    return _from_torch(res, to_dtype)


def nanpercentile(a: Any, q: Any, axis: Union[None, int, Iterable[int]] = None, out: Optional[ndarray] = None,
                  overwrite_input: bool = False, method: str = "linear", keepdims: bool = False) -> ndarray:
    """The q-th percentile(s), ignoring NaNs: ``nanquantile`` with ``q / 100``
    (reference: cunumeric/module.py:8965-9065)."""
    q_arr = np.true_divide(np.asarray(q, dtype=np.float64), 100.0)
    if q_arr.size and not (np.all(q_arr >= 0) and np.all(q_arr <= 1)):
        raise ValueError("Percentiles must be in the range [0, 100]")
    return nanquantile(a, q_arr, axis=axis, out=out, overwrite_input=overwrite_input, method=method,
                       keepdims=keepdims)
