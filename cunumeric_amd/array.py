"""``ndarray``: a dense, row-major device array with the sort-family methods.

Counterpart of the pieces of the reference's ndarray / DeferredArray that the sort path
touches: ``ndarray.sort / argsort / partition / argpartition``
(cunumeric/array.py:3710-3759, 3360-3420), ``DeferredArray.sort / partition``
(cunumeric/deferred.py:3535-3578) and the helpers ``sort.py`` calls on a thunk:
``reshape``, ``swapaxes`` + deep ``copy`` (deferred.py:1121+, 1333-1346, 392-401).
Array-likes are converted on entry the way ``add_boilerplate`` does
(cunumeric/array.py:86-149).
"""
from __future__ import annotations

from typing import Any, Optional, Sequence, Union

import numpy as np
import torch

from . import _lib
from .config import MAX_DIM, to_core_dtype
from .runtime import runtime
from .sort import sort as _sort_frontend

_TORCH_TO_NUMPY = {
    torch.bool: np.bool_,
    torch.int8: np.int8,
    torch.int16: np.int16,
    torch.int32: np.int32,
    torch.int64: np.int64,
    torch.uint8: np.uint8,
    torch.uint16: np.uint16,
    torch.uint32: np.uint32,
    torch.uint64: np.uint64,
    torch.float16: np.float16,
    torch.float32: np.float32,
    torch.float64: np.float64,
    torch.complex64: np.complex64,
    torch.complex128: np.complex128,
}


class _Flags:
    def __init__(self, writeable: bool = True):
        self.writeable = writeable
        self.c_contiguous = True


def check_writeable(arr: "ndarray") -> None:
    """(reference: cunumeric/array.py ``check_writeable``)"""
    if not arr.flags.writeable:
        raise ValueError("array is not writeable")


def _reject_order(order, what: str) -> None:
    """Structured-array field names have no meaning here (reference: cunumeric/deferred.py:3549-3553)."""
    if order is not None:
        raise NotImplementedError(f"{what}: 'order' is not supported, arrays hold plain numeric values")


def _check_axis(axis, ndim: int) -> None:
    if axis is not None and not -ndim <= axis < ndim:
        raise ValueError(f"axis {axis} is out of bounds for an array of dimension {ndim}")


class ndarray:
    """Dense C-ordered array in device memory (one HBM allocation, byte-addressed)."""

    __array_priority__ = 100

    def __init__(self, shape, dtype=np.float64, _buf: Optional[torch.Tensor] = None):
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        self._shape = tuple(int(s) for s in shape)
        self._dtype = np.dtype(dtype)
        to_core_dtype(self._dtype)  # TypeError for unsupported dtypes
        if len(self._shape) > MAX_DIM:
            raise ValueError(f"at most {MAX_DIM} dimensions are supported")
        nbytes = self.size * self._dtype.itemsize
        self._buf = _buf if _buf is not None else runtime.alloc_bytes(nbytes)
        self.flags = _Flags()

    # ---- basic properties -------------------------------------------------------------
    @property
    def shape(self):
        return self._shape

    @property
    def dtype(self):
        return self._dtype

    @property
    def ndim(self) -> int:
        return len(self._shape)

    @property
    def size(self) -> int:
        n = 1
        for s in self._shape:
            n *= s
        return n

    @property
    def nbytes(self) -> int:
        return self.size * self._dtype.itemsize

    def _ptr(self) -> int:
        return self._buf.data_ptr()

    def __len__(self) -> int:
        if self.ndim == 0:
            raise TypeError("len() of unsized object")
        return self._shape[0]

    def __repr__(self) -> str:
        return f"cunumeric_amd.ndarray(shape={self._shape}, dtype={self._dtype})"

    # ---- conversion -------------------------------------------------------------------
    def __array__(self, dtype=None, copy=None):
        torch.cuda.current_stream().synchronize()
        out = runtime.download(self._buf, self._shape, self._dtype)
        return out.astype(dtype) if dtype is not None else out

    def to_torch(self) -> torch.Tensor:
        """Zero-copy view of the buffer as a torch tensor of the matching dtype."""
        for t, n in _TORCH_TO_NUMPY.items():
            if np.dtype(n) == self._dtype:
                return self._buf[: self.nbytes].view(t).reshape(self._shape)
        raise TypeError(self._dtype)

    def astype(self, dtype, copy: bool = True) -> "ndarray":
        dtype = np.dtype(dtype)
        if dtype == self._dtype and not copy:
            return self
        # dtype conversion is not part of the sort path: done through torch on the device
        src = self.to_torch()
        for t, n in _TORCH_TO_NUMPY.items():
            if np.dtype(n) == dtype:
                dst = src.to(t).contiguous()
                return ndarray(self._shape, dtype, _buf=dst.reshape(-1).view(torch.uint8))
        raise TypeError(f"cuNumeric does not support dtype={dtype}")

    def copy(self) -> "ndarray":
        return ndarray(self._shape, self._dtype, _buf=self._buf.clone())

    # ---- helpers used by the sort front-end -------------------------------------------
    def _empty_like_shape(self, shape) -> "ndarray":
        """(reference: runtime.create_empty_thunk, cunumeric/runtime.py:448-460)"""
        return ndarray(shape, self._dtype)

    def _rebind(self, other: "ndarray") -> None:
        """Take over another array's storage: what ``output.base = ...`` does in the
        reference front-end (cunumeric/sort.py:43-44, 75-83)."""
        assert other._dtype == self._dtype
        self._buf = other._buf
        self._shape = other._shape

    def reshape(self, shape) -> "ndarray":
        """Dense row-major arrays reshape without moving data."""
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        shape = tuple(int(s) for s in shape)
        n = 1
        for s in shape:
            n *= s
        if n != self.size:
            raise ValueError(f"cannot reshape array of size {self.size} into shape {shape}")
        return ndarray(shape, self._dtype, _buf=self._buf)

    def _swap_with_last(self, axis: int) -> "ndarray":
        """Dense copy with ``axis`` and the last axis exchanged: ``swapaxes`` followed by
        the deep copy of cunumeric/sort.py:57-65."""
        nd = self.ndim
        shp = self._shape
        new_shape = list(shp)
        new_shape[axis], new_shape[nd - 1] = shp[nd - 1], shp[axis]
        out = ndarray(tuple(new_shape), self._dtype)
        if self.size == 0:
            return out
        outer = 1
        for s in shp[:axis]:
            outer *= s
        mid = 1
        for s in shp[axis + 1 : nd - 1]:
            mid *= s
        _lib.check(
            _lib.load().misort_swap_last(
                self._ptr(), out._ptr(), outer, shp[axis], mid, shp[nd - 1],
                self._dtype.itemsize, runtime.stream_handle(),
            )
        )
        return out

    # ---- the thunk-level sort (DeferredArray.sort / partition) ------------------------
    def _thunk_sort(
        self,
        rhs: "ndarray",
        argsort: bool = False,
        axis: Union[int, None] = -1,
        kind: str = "quicksort",
        order: Union[None, str, list] = None,
    ) -> None:
        """Same contract as the reference's thunk (cunumeric/deferred.py:3535-3557): only
        the literal kind "stable" asks for stability, field names cannot be given (arrays
        hold plain numbers), an axis outside the array is a ValueError."""
        _reject_order(order, "sort")
        _check_axis(axis, rhs.ndim)
        _sort_frontend(self, rhs, argsort, axis, kind == "stable")

    def _thunk_partition(
        self,
        rhs: "ndarray",
        kth: Union[int, Sequence[int]],
        argpartition: bool = False,
        axis: Union[int, None] = -1,
        kind: str = "introselect",
        order: Union[None, str, list] = None,
    ) -> None:
        """(reference: cunumeric/deferred.py:3559-3578, which does not look at ``kth`` and
        sorts.  Here a single in-range ``kth`` selects instead of sorting; a sequence of
        positions or an out-of-range one sorts, as the reference always does.)"""
        _reject_order(order, "partition")
        _check_axis(axis, rhs.ndim)

        k: Optional[int] = None
        if isinstance(kth, (int, np.integer)) and not isinstance(kth, bool):
            n = rhs.size if axis is None else (rhs.shape[axis] if rhs.ndim else 1)
            k = int(kth) + (n if int(kth) < 0 else 0)
            if not 0 <= k < n:
                k = None
        _sort_frontend(self, rhs, argpartition, axis, False, k)

    # ---- public methods ---------------------------------------------------------------
    def sort(self, axis: Any = -1, kind: str = "quicksort", order=None) -> None:
        """a.sort(axis=-1, kind=None, order=None): sort in place
        (reference: cunumeric/array.py:3710-3732)."""
        check_writeable(self)
        self._thunk_sort(rhs=self, axis=axis, kind=kind, order=order)

    def argsort(self, axis: Any = -1, kind: str = "quicksort", order=None) -> "ndarray":
        """(reference: cunumeric/array.py:3734-3759)"""
        result = ndarray(self.shape, np.int64)
        result._thunk_sort(rhs=self, argsort=True, axis=axis, kind=kind, order=order)
        return result

    def partition(self, kth, axis: Any = -1, kind: str = "introselect", order=None) -> None:
        """(reference: cunumeric/array.py:3360-3386)"""
        check_writeable(self)
        self._thunk_partition(rhs=self, kth=kth, axis=axis, kind=kind, order=order)

    def argpartition(self, kth, axis: Any = -1, kind: str = "introselect", order=None) -> "ndarray":
        """(reference: cunumeric/array.py:3388-3420)"""
        result = ndarray(self.shape, np.int64)
        result._thunk_partition(
            rhs=self, argpartition=True, kth=kth, axis=axis, kind=kind, order=order
        )
        return result


    def take(self, indices: "ndarray") -> "ndarray":
        """Elements of a 1-D array at integer positions (what ``a.take(sorter)`` needs in
        searchsorted, reference cunumeric/array.py:3701; indexing is not part of the sort
        path and goes through torch on the device)."""
        if self.ndim != 1:
            raise ValueError("take: only 1-D arrays are supported here")
        idx = indices.to_torch().to(torch.int64).reshape(-1)
        es = self._dtype.itemsize
        rows = self._buf[: self.nbytes].reshape(self.size, es)
        return ndarray(indices.shape, self._dtype, _buf=rows[idx].reshape(-1).contiguous())

    def searchsorted(self, v: Any, side: str = "left", sorter: Optional["ndarray"] = None):
        """a.searchsorted(v, side='left', sorter=None): insertion indices that keep ``a``
        sorted; int64 of v's shape, a Python int for a scalar v
        (reference: cunumeric/array.py:3637-3709, cunumeric/deferred.py:3511-3533)."""
        if self.ndim != 1:
            raise ValueError("Dimension mismatch: self must be a 1D array")
        if side not in ("left", "right"):
            raise ValueError(f"side must be 'left' or 'right', not {side!r}")
        scalar = np.ndim(v) == 0 and not isinstance(v, (ndarray, torch.Tensor))
        queries = convert_to_cunumeric_ndarray(v)  # a Python scalar becomes a 0-d array
        a = self
        # the kernel compares one element type: promote both sides to their common type
        common = np.result_type(a.dtype, queries.dtype)
        if queries.dtype != common:
            queries = queries.astype(common)
        if a.dtype != common:
            a = a.astype(common)
        if sorter is not None and a.shape[0] > 1:
            perm = convert_to_cunumeric_ndarray(sorter)
            if perm.ndim != 1:
                raise ValueError("sorter must be one-dimensional")
            if perm.shape != a.shape:
                raise ValueError("sorter must have as many elements as the array it sorts")
            if not np.issubdtype(perm.dtype, np.integer):
                raise ValueError("sorter must hold integers")
            a = a.take(perm)
        v_ndarray = queries
        result = ndarray(v_ndarray.shape, np.int64)
        if v_ndarray.size:
            lib = _lib.load()
            code = to_core_dtype(a.dtype)
            # many queries into a large array: the library sorts the queries first (workspace)
            need = lib.misort_searchsorted_scratch_bytes(code, a.size, v_ndarray.size)
            scratch = runtime.alloc_bytes(need) if need else None
            _lib.check(
                lib.misort_searchsorted_ws(
                    code, a._ptr() if a.size else None, a.size, v_ndarray._ptr(), v_ndarray.size,
                    int(side == "left"), result._ptr(), scratch.data_ptr() if need else None, need,
                    runtime.stream_handle(),
                )
            )
        if scalar:
            return int(np.asarray(result).reshape(-1)[0])
        return result


    def unique(self) -> "ndarray":
        """a.unique(): the sorted distinct elements of the flattened array.  The result's
        length is only known on the device, so this synchronises the stream, as the
        reference's unbound output store does
        (reference: cunumeric/array.py:4155-4172, cunumeric/deferred.py:3490-3508)."""
        n = self.size
        if n == 0:
            return ndarray((0,), self._dtype)
        lib = _lib.load()
        code = to_core_dtype(self._dtype)
        need = lib.misort_unique_scratch_bytes(code, n)
        scratch = runtime.alloc_bytes(need)
        out = ndarray((n,), self._dtype)
        count = torch.zeros(1, dtype=torch.int64, device=runtime.device())
        _lib.check(
            lib.misort_unique(code, self._ptr(), out._ptr(), count.data_ptr(), n, scratch.data_ptr(),
                              need, runtime.stream_handle())
        )
        k = int(count.item())  # synchronises
        del scratch
        es = self._dtype.itemsize
        return ndarray((k,), self._dtype, _buf=out._buf[: k * es].clone() if k else None)


def convert_to_cunumeric_ndarray(obj: Any) -> ndarray:
    """Array-like -> device ndarray (reference: cunumeric/array.py
    ``convert_to_cunumeric_ndarray`` used by ``add_boilerplate`` :86-149)."""
    if isinstance(obj, ndarray):
        return obj
    if isinstance(obj, torch.Tensor):
        np_dtype = _TORCH_TO_NUMPY.get(obj.dtype)
        if np_dtype is None:
            raise TypeError(f"cuNumeric does not support dtype={obj.dtype}")
        t = obj.detach().contiguous()
        if not t.is_cuda:
            t = t.to(runtime.device())
        if t.numel() == 0:
            return ndarray(tuple(t.shape), np_dtype)
        buf = t.reshape(-1).view(torch.uint8)
        if t.data_ptr() == obj.data_ptr():
            buf = buf.clone()  # never alias the caller's tensor
        return ndarray(tuple(t.shape), np_dtype, _buf=buf)
    a = np.asarray(obj)
    to_core_dtype(a.dtype)
    return ndarray(a.shape, a.dtype, _buf=runtime.upload(a))


def array(obj: Any, dtype=None) -> ndarray:
    if dtype is not None and not isinstance(obj, (ndarray, torch.Tensor)):
        obj = np.asarray(obj, dtype=dtype)
    out = convert_to_cunumeric_ndarray(obj)
    if dtype is not None and np.dtype(dtype) != out.dtype:
        out = out.astype(dtype)
    return out


asarray = array
