"""ctypes binding of libmisort.so (the C ABI declared in include/misort.h).

The library is loaded from the package directory only.  There is no fallback: if the
shared object is missing, every call raises ``MisortLibraryError``.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmisort.so")

# every symbol include/misort.h declares
EXPORTS = (
    "misort_version",
    "misort_dtype_size",
    "misort_last_error",
    "misort_scratch_bytes",
    "misort_local",
    "misort_local_profiled",
    "misort_kernel_name",
    "misort_describe_plan",
    "misort_swap_last",
    "misort_scratch_bytes_chunked",
    "misort_local_chunked",
    "misort_local_static",
    "misort_selftest_lds_lane_order",
    "misort_searchsorted",
    "misort_searchsorted_scratch_bytes",
    "misort_searchsorted_ws",
    "misort_unique_scratch_bytes",
    "misort_unique",
    "misort_partition_scratch_bytes",
    "misort_partition",
    "misort_select_scratch_bytes",
    "misort_select",
    "misort_sort_axis",
    "misort_scratch_bytes_opts",
    "misort_local_opts",
    "misort_describe_plan_opts",
    "misort_init",
    "misort_rank_mode",
)

STATUS_NAMES = {
    0: "MISORT_OK",
    1: "MISORT_ERR_DTYPE",
    2: "MISORT_ERR_NULL",
    3: "MISORT_ERR_SHAPE",
    4: "MISORT_ERR_SCRATCH",
    5: "MISORT_ERR_ALIGN",
    6: "MISORT_ERR_RUNTIME",
    7: "MISORT_ERR_ALIAS",
    8: "MISORT_ERR_UNSUPPORTED",
}


class Options(ctypes.Structure):
    """misort_options of include/misort.h; the defaults mean "as misort_local"."""

    _fields_ = [("target_chunks", c_size_t), ("early_last_min_bytes", ctypes.c_longlong),
                ("bucket_path", c_int), ("bucket_bins", ctypes.c_uint), ("bucket_cap", ctypes.c_uint),
                ("low_cardinality", c_int), ("bucket_oversample", ctypes.c_uint), ("counting_sort", c_int), ("upper_first", c_int)]

    def __init__(self, target_chunks=0, early_last_min_bytes=-1, bucket_path=-1, bucket_bins=0, bucket_cap=0,
                 low_cardinality=-1, bucket_oversample=0, counting_sort=-1, upper_first=-1):
        super().__init__(target_chunks, early_last_min_bytes, bucket_path, bucket_bins, bucket_cap, low_cardinality,
                         bucket_oversample, counting_sort, upper_first)


class MisortLibraryError(RuntimeError):
    """libmisort.so is missing or cannot be loaded."""


class MisortError(RuntimeError):
    """A libmisort entry point returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


_lib = None


def load():
    """Load libmisort.so once and declare the argument types of every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MisortLibraryError(
            f"{LIB_PATH} not found: build it with cunumeric_amd/csrc/build.sh "
            "(or __graft_entry__.build()); there is no CPU fallback"
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise MisortLibraryError(f"cannot load {LIB_PATH}: {e}") from e

    lib.misort_version.restype = c_int
    lib.misort_version.argtypes = []
    lib.misort_dtype_size.restype = c_size_t
    lib.misort_dtype_size.argtypes = [c_int]
    lib.misort_last_error.restype = c_char_p
    lib.misort_last_error.argtypes = []
    lib.misort_scratch_bytes.restype = c_size_t
    lib.misort_scratch_bytes.argtypes = [c_int, c_size_t, c_size_t, c_int, c_int]
    lib.misort_local.restype = c_int
    lib.misort_local.argtypes = [
        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int64,
        c_void_p, c_size_t, c_void_p,
    ]
    lib.misort_local_profiled.restype = c_int
    lib.misort_local_profiled.argtypes = [
        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int64,
        c_void_p, c_size_t, c_void_p,
        ctypes.POINTER(ctypes.c_float), ctypes.POINTER(c_int), c_int, ctypes.POINTER(c_int),
    ]
    lib.misort_kernel_name.restype = c_char_p
    lib.misort_kernel_name.argtypes = [c_int]
    lib.misort_describe_plan.restype = c_int
    lib.misort_describe_plan.argtypes = [c_int, c_size_t, c_size_t, c_int, c_int, c_char_p, c_size_t]
    lib.misort_searchsorted_scratch_bytes.restype = c_size_t
    lib.misort_searchsorted_scratch_bytes.argtypes = [c_int, c_size_t, c_size_t]
    lib.misort_searchsorted_ws.restype = c_int
    lib.misort_searchsorted_ws.argtypes = [c_int, c_void_p, c_size_t, c_void_p, c_size_t, c_int, c_void_p,
                                           c_void_p, c_size_t, c_void_p]
    lib.misort_searchsorted.restype = c_int
    lib.misort_searchsorted.argtypes = [c_int, c_void_p, c_size_t, c_void_p, c_size_t, c_int, c_void_p,
                                        c_void_p]
    lib.misort_unique_scratch_bytes.restype = c_size_t
    lib.misort_unique_scratch_bytes.argtypes = [c_int, c_size_t]
    lib.misort_unique.restype = c_int
    lib.misort_unique.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t,
                                  c_void_p]
    lib.misort_partition_scratch_bytes.restype = c_size_t
    lib.misort_partition_scratch_bytes.argtypes = [c_int, c_size_t, c_size_t, c_int, ctypes.c_longlong]
    lib.misort_partition.restype = c_int
    lib.misort_partition.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t,
                                     ctypes.c_longlong, c_int64, c_void_p, c_size_t, c_void_p]
    lib.misort_select_scratch_bytes.restype = c_size_t
    lib.misort_select_scratch_bytes.argtypes = [c_int, c_size_t, c_size_t, ctypes.c_longlong]
    lib.misort_select.restype = c_int
    lib.misort_select.argtypes = [c_int, c_void_p, c_size_t, c_size_t, ctypes.c_longlong, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_size_t, c_void_p]
    lib.misort_sort_axis.restype = c_int
    lib.misort_sort_axis.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t,
                                     c_int64, c_void_p]
    lib.misort_scratch_bytes_chunked.restype = c_size_t
    lib.misort_scratch_bytes_chunked.argtypes = [c_int, c_size_t, c_size_t, c_int, c_int, c_size_t]
    lib.misort_local_chunked.restype = c_int
    lib.misort_local_chunked.argtypes = [
        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int64,
        c_void_p, c_size_t, c_void_p, c_size_t,
    ]
    lib.misort_scratch_bytes_opts.restype = c_size_t
    lib.misort_scratch_bytes_opts.argtypes = [c_int, c_size_t, c_size_t, c_int, c_int, ctypes.POINTER(Options)]
    lib.misort_local_opts.restype = c_int
    lib.misort_local_opts.argtypes = [
        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int64,
        c_void_p, c_size_t, c_void_p, ctypes.POINTER(Options),
    ]
    lib.misort_describe_plan_opts.restype = c_int
    lib.misort_describe_plan_opts.argtypes = [c_int, c_size_t, c_size_t, c_int, c_int, ctypes.POINTER(Options),
                                              c_char_p, c_size_t]
    lib.misort_init.restype = c_int
    lib.misort_init.argtypes = []
    lib.misort_rank_mode.restype = c_int
    lib.misort_rank_mode.argtypes = []
    lib.misort_local_static.restype = c_int
    lib.misort_local_static.argtypes = [
        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int64, c_void_p,
    ]
    lib.misort_selftest_lds_lane_order.restype = c_int
    lib.misort_selftest_lds_lane_order.argtypes = [ctypes.c_uint, ctypes.POINTER(ctypes.c_ulonglong),
                                                   ctypes.POINTER(ctypes.c_ulonglong), c_void_p]
    lib.misort_swap_last.restype = c_int
    lib.misort_swap_last.argtypes = [
        c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_size_t, c_size_t, c_void_p,
    ]
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != 0:
        raise MisortError(status, load().misort_last_error().decode())


def describe_plan(dtype_code: int, volume: int, sort_dim_size: int, argsort: bool,
                  has_indices_in: bool = False, options: "Options | None" = None) -> str:
    lib = load()
    buf = ctypes.create_string_buffer(512)
    if options is None:
        check(lib.misort_describe_plan(dtype_code, volume, sort_dim_size, int(argsort),
                                       int(has_indices_in), buf, len(buf)))
    else:
        check(lib.misort_describe_plan_opts(dtype_code, volume, sort_dim_size, int(argsort),
                                            int(has_indices_in), ctypes.byref(options), buf, len(buf)))
    return buf.value.decode()
