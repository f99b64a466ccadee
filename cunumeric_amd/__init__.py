"""cunumeric_amd: the single-GPU sort path of cuNumeric, native to MI355X (gfx950).

``import cunumeric_amd as num`` gives the sort family of ``cunumeric``:
``num.sort, num.argsort, num.msort, num.sort_complex, num.partition, num.argpartition,
num.searchsorted, num.digitize, num.unique, num.quantile, num.percentile, num.nanquantile, num.nanpercentile``
and ``ndarray.sort / argsort / partition / argpartition``, backed by hand-written HIP
kernels in libmisort.so (C ABI in include/misort.h).
"""
from .array import array, asarray, ndarray
from .module import argpartition, argsort, digitize, msort, partition, searchsorted, sort, sort_complex, unique
from .quantile import nanpercentile, nanquantile, percentile, quantile

__all__ = [
    "array", "asarray", "ndarray",
    "argpartition", "argsort", "digitize", "msort", "partition", "searchsorted", "sort", "sort_complex", "unique",
    "nanpercentile", "nanquantile", "percentile", "quantile",
]
__version__ = "0.1.0"
