"""SORT front-end: axis handling and task construction.

Mirrors cunumeric/sort.py of the reference function by function:
``sort`` (:118-136), ``sort_flattened`` (:30-44), ``sort_swapped`` (:47-83),
``sort_task`` (:86-115).  Where the reference hands a task to Legate, ``sort_task``
here fills the same record (one input, one aligned output, scalars
``[argsort, shape, stable]``) and executes it on the C ABI of libmisort.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Optional, Union

import numpy as np
from numpy.lib.array_utils import normalize_axis_index

from . import _lib
from .config import CuNumericOpCode, to_core_dtype
from .runtime import runtime

if TYPE_CHECKING:
    from .array import ndarray


@dataclass
class SortTask:
    """The SORT task record: what ``sort_template`` unpacks from the TaskContext
    (src/cunumeric/sort/sort_template.inl:86-107): inputs()[0], outputs()[0],
    scalars()[0] = argsort, scalars()[1] = global shape, scalars()[2] = stable.
    Stores are dense and row-major, as the mapper demands for this task
    (src/cunumeric/mapper.cc:181-196)."""

    op: CuNumericOpCode = CuNumericOpCode.SORT
    inputs: list = field(default_factory=list)
    outputs: list = field(default_factory=list)
    scalars: list = field(default_factory=list)
    # partition only (no counterpart in the reference's task): position to partition around
    kth: Optional[int] = None

    def add_input(self, store: "ndarray") -> None:
        self.inputs.append(store)

    def add_output(self, store: "ndarray") -> None:
        self.outputs.append(store)

    def add_alignment(self, a: "ndarray", b: "ndarray") -> None:
        if a.shape != b.shape:
            raise ValueError("aligned stores must have the same shape")

    def add_scalar_arg(self, value) -> None:
        self.scalars.append(value)

    def execute(self) -> None:
        """The single-GPU body of SortImpl / SortImplBody<GPU>
        (sort_template.inl:42-84, sort.cu:1661-1753): volume, segment size of the last
        axis, early-out on an empty rectangle, then the local sort."""
        inp, out = self.inputs[0], self.outputs[0]
        argsort, shape, stable = self.scalars
        shape = tuple(int(s) for s in shape)
        volume = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        segment_size = shape[-1] if len(shape) else 1
        if volume == 0:
            return
        lib = _lib.load()
        code = to_core_dtype(inp.dtype)
        if self.kth is not None:
            # partition / argpartition around one position: selection instead of a sort
            need = lib.misort_partition_scratch_bytes(code, volume, segment_size, int(argsort), self.kth)
            scratch = runtime.alloc_bytes(need)
            _lib.check(
                lib.misort_partition(
                    code, inp._ptr(), None if argsort else out._ptr(), out._ptr() if argsort else None,
                    volume, segment_size, self.kth, 0, scratch.data_ptr(), need,
                    runtime.stream_handle(),
                )
            )
            del scratch
            return
        need = lib.misort_scratch_bytes(code, volume, segment_size, int(argsort), 0)
        scratch = runtime.alloc_bytes(need)
        if argsort:
            values_out, indices_out = None, out._ptr()
        else:
            values_out, indices_out = out._ptr(), None
        _lib.check(
            lib.misort_local(
                code, inp._ptr(), values_out, None, indices_out, volume, segment_size,
                int(stable), 0, scratch.data_ptr(), need, runtime.stream_handle(),
            )
        )
        # the stream orders later work after the sort; scratch is returned to the
        # caching allocator, which keeps it tied to this stream
        del scratch


def sort_flattened(output: "ndarray", input: "ndarray", argsort: bool, stable: bool,
                   kth: Optional[int] = None) -> None:
    flattened = input.reshape((input.size,))
    sort_result = output._empty_like_shape(flattened.shape)
    sort(sort_result, flattened, argsort, stable=stable, kth=kth)
    output._rebind(sort_result)


def sort_swapped(
    output: "ndarray", input: "ndarray", argsort: bool, sort_axis: int, stable: bool,
    kth: Optional[int] = None,
) -> None:
    sort_axis = normalize_axis_index(sort_axis, input.ndim)
    # dense copy with the sort axis last
    swapped_copy = input._swap_with_last(sort_axis)
    if argsort:
        sort_result = output._empty_like_shape(swapped_copy.shape)
        sort(sort_result, swapped_copy, argsort, stable=stable, kth=kth)
        output._rebind(sort_result._swap_with_last(sort_axis))
    elif swapped_copy.dtype.itemsize == 8 and swapped_copy.size >= (1 << 25) and kth is None:
        # long sorts of 8-byte keys are quicker out of place: the library then tries the radix
        # passes over the upper bytes only first, which it cannot do where the result
        # overwrites the input (the reference sorts the copy in place, cunumeric/sort.py:62-70)
        sort_result = output._empty_like_shape(swapped_copy.shape)
        sort(sort_result, swapped_copy, argsort, stable=stable, kth=kth)
        del swapped_copy
        output._rebind(sort_result._swap_with_last(sort_axis))
    else:
        sort(swapped_copy, swapped_copy, argsort, stable=stable, kth=kth)
        output._rebind(swapped_copy._swap_with_last(sort_axis))


MISORT_ERR_UNSUPPORTED = 8


def sort_along_axis(output: "ndarray", input: "ndarray", argsort: bool, sort_axis: int) -> bool:
    """Short sort axes that are not the last one: sort the columns where they lie instead of
    the two transposed copies of ``sort_swapped`` (no counterpart in the reference, which
    always swaps: cunumeric/sort.py:47-83).  Returns False when the library does not serve
    the shape; the caller then swaps."""
    shape = input.shape
    outer = int(np.prod(shape[:sort_axis], dtype=np.int64))
    k = int(shape[sort_axis])
    inner = int(np.prod(shape[sort_axis + 1:], dtype=np.int64))
    if inner == 1 or k > 1024:
        return False
    lib = _lib.load()
    result = output._empty_like_shape(shape)
    if input.size:
        rc = lib.misort_sort_axis(
            to_core_dtype(input.dtype), input._ptr(), None if argsort else result._ptr(),
            result._ptr() if argsort else None, outer, k, inner, 0, runtime.stream_handle(),
        )
        if rc == MISORT_ERR_UNSUPPORTED:
            return False
        _lib.check(rc)
    output._rebind(result)
    return True


def sort_task(output: "ndarray", input: "ndarray", argsort: bool, stable: bool,
              kth: Optional[int] = None) -> None:
    task = SortTask()
    task.kth = kth
    task.add_input(input)
    task.add_output(output)
    task.add_alignment(output, input)
    task.add_scalar_arg(argsort)
    task.add_scalar_arg(input.shape)
    task.add_scalar_arg(stable)
    task.execute()


def sort(
    output: "ndarray",
    input: "ndarray",
    argsort: bool,
    axis: Union[int, None] = -1,
    stable: bool = False,
    kth: Optional[int] = None,
) -> None:
    """``kth`` (not in the reference, which sorts for partition): a position along the sort
    axis; when given, the rows are only partitioned around it."""
    if axis is None and input.ndim > 1:
        # no axis: the array is sorted as one flat row
        sort_flattened(output, input, argsort, stable, kth)
        return
    ax = 0 if axis is None else normalize_axis_index(axis, input.ndim)
    if ax == input.ndim - 1:
        sort_task(output, input, argsort, stable, kth)       # rows are contiguous: sort them
    elif not sort_along_axis(output, input, argsort, ax):     # short axis: sorted where it lies
        sort_swapped(output, input, argsort, ax, stable, kth)  # else through a transposed copy
