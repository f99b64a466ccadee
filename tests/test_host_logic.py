"""CPU-only checks: the C-ABI library loads and exports what include/misort.h declares,
argument validation answers before any GPU work, and the plan / scratch queries are sane."""
import ctypes
import os
import re

import numpy as np
import pytest

from cunumeric_amd import _lib
from cunumeric_amd.config import SUPPORTED_DTYPES, CuNumericOpCode, to_core_dtype

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "misort.h")).read()
    declared = set(re.findall(r"\b(misort_[a-z_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name


def test_version_and_dtype_sizes(lib):
    assert lib.misort_version() >= 100
    for dt, code in SUPPORTED_DTYPES.items():
        assert lib.misort_dtype_size(code) == dt.itemsize
    assert lib.misort_dtype_size(14) == 0 and lib.misort_dtype_size(-1) == 0


def test_dtype_table_matches_reference_order():
    names = ["bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64",
             "float16", "float32", "float64", "complex64", "complex128"]
    assert [np.dtype(d).name for d in SUPPORTED_DTYPES] == names
    assert list(SUPPORTED_DTYPES.values()) == list(range(14))
    with pytest.raises(TypeError):
        to_core_dtype(np.dtype("U3"))
    assert CuNumericOpCode.SORT.name == "SORT"


def test_scratch_query(lib):
    assert lib.misort_scratch_bytes(10, 0, 0, 1, 0) == 0
    assert lib.misort_scratch_bytes(99, 100, 100, 1, 0) == 0  # bad dtype
    small = lib.misort_scratch_bytes(10, 256 * 1024, 256, 0, 0)  # row kernels: no buffers
    assert 0 < small <= 4096
    n = 1 << 24
    need = lib.misort_scratch_bytes(10, n, n, 1, 0)
    # two key buffers + two 32-bit payload buffers + per-chunk tables
    assert 16 * n <= need <= 16 * n + (64 << 20)
    need64 = lib.misort_scratch_bytes(10, n, n, 1, 1)  # caller payload: int64 carried
    assert need64 > need


def test_describe_plan(lib):
    assert "strategy=radix" in _lib.describe_plan(10, 1 << 28, 1 << 28, True)
    assert "passes=4" in _lib.describe_plan(10, 1 << 28, 1 << 28, True)
    assert "payload=idx32" in _lib.describe_plan(10, 1 << 28, 1 << 28, True)
    assert "strategy=row_wave" in _lib.describe_plan(11, 1 << 20, 256, False)
    assert "strategy=row_block" in _lib.describe_plan(11, 1 << 20, 4096, False)
    assert "passes=8" in _lib.describe_plan(4, 1 << 28, 1 << 28, True)
    assert "passes=16" in _lib.describe_plan(13, 1 << 20, 1 << 20, True)
    assert "strategy=count16" in _lib.describe_plan(9, 1 << 30, 1 << 30, False)  # values only
    assert "passes=2" in _lib.describe_plan(9, 1 << 30, 1 << 30, True)
    assert "passes=2" in _lib.describe_plan(9, 1 << 22, 1 << 21, False)  # two rows: radix


def test_plans_of_the_paths_beside_the_radix_passes(lib):
    """Where the four-launch path, the counting sort and the two attempts of long radix sorts
    are planned (type codes of include/misort.h: 1 int8, 2 int16, 3 int32, 4 int64, 9 float16,
    10 float32, 11 float64, 12 complex64, 13 complex128)."""
    from cunumeric_amd._lib import Options

    plan = _lib.describe_plan
    bucket = lambda code, vol, row, arg, **kw: "strategy=bucket" in plan(code, vol, row, arg, **kw)
    # medium rows: four launches, up to where the radix passes catch up
    assert bucket(3, 1 << 20, 1 << 20, False) and bucket(3, 1 << 21, 1 << 21, True)
    assert not bucket(3, (1 << 21) + 1, (1 << 21) + 1, False)
    assert bucket(3, 3 << 19, 3 << 16, True) and not bucket(3, 1 << 21, 1 << 18, True)   # several rows
    assert bucket(11, 1 << 21, 1 << 21, True) and bucket(4, 1 << 22, 1 << 19, False)
    assert not bucket(4, 1 << 23, 1 << 19, False)
    assert bucket(2, 1 << 19, 1 << 19, False) and not bucket(2, 1 << 20, 1 << 20, False)
    assert bucket(9, 1 << 20, 1 << 20, False) and not bucket(9, 1 << 19, 1 << 19, True)
    assert not bucket(1, 1 << 16, 1 << 16, True) and not bucket(13, 1 << 16, 1 << 16, True)
    assert bucket(1, 1 << 16, 1 << 16, True, options=Options(bucket_path=1))
    assert not bucket(3, 1 << 18, 1 << 18, False, options=Options(bucket_path=0))
    assert "bin_cap=16384" in plan(4, 1 << 20, 1 << 20, True)
    # counting sort of 2-byte values
    assert "strategy=count16" in plan(9, 1 << 24, 1 << 24, False)
    assert "strategy=count16" not in plan(2, 1 << 24, 1 << 24, False)
    assert "strategy=count16" in plan(2, 1 << 26, 1 << 26, False)
    assert "strategy=count16" in plan(2, 1 << 20, 1 << 20, False, options=Options(counting_sort=1))
    assert "strategy=count16" not in plan(2, 1 << 26, 1 << 26, False, options=Options(counting_sort=0))
    # long radix sorts: few distinct keys, and 8-byte keys by their upper bytes first
    assert "low_cardinality_attempt=1" in plan(10, 1 << 27, 1 << 27, True)
    assert "low_cardinality_attempt" not in plan(10, 1 << 26, 1 << 26, True)
    assert "upper_first_attempt=1" in plan(11, 1 << 25, 1 << 25, False)
    assert "upper_first_attempt=1" in plan(12, 1 << 26, 1 << 20, True)
    assert "upper_first_attempt" not in plan(11, (1 << 25) - 1, (1 << 25) - 1, False)
    assert "upper_first_attempt" not in plan(10, 1 << 28, 1 << 28, True)
    assert "upper_first_attempt" not in plan(13, 1 << 26, 1 << 26, True)
    assert "upper_first_attempt=2" in plan(4, 1 << 22, 1 << 22, True, options=Options(bucket_path=0, upper_first=2))
    assert "upper_first_attempt" not in plan(4, 1 << 26, 1 << 26, True, options=Options(upper_first=0))
    # the attempt's fix-up needs the keys of an argsort's result: 8 bytes per element more scratch
    n = 1 << 26
    with_keys = lib.misort_scratch_bytes(4, n, n, 1, 0)
    import ctypes
    o = Options(upper_first=0)
    without = lib.misort_scratch_bytes_opts(4, n, n, 1, 0, ctypes.byref(o))
    assert 8 * n <= with_keys - without <= 8 * n + 4096


def test_argument_errors_need_no_gpu(lib):
    def call(dtype, vin, vout, iin, iout, volume, row, scratch, sbytes):
        return lib.misort_local(dtype, vin, vout, iin, iout, volume, row, 1, 0, scratch, sbytes, None)

    assert call(10, None, None, None, None, 0, 0, None, 0) == 0  # empty: nothing to do
    assert call(77, 256, 256, None, None, 8, 8, 256, 1 << 20) == 1  # MISORT_ERR_DTYPE
    assert call(10, 256, 256, None, None, 10, 3, 256, 1 << 20) == 3  # MISORT_ERR_SHAPE
    assert "multiple" in lib.misort_last_error().decode()
    assert call(10, None, 256, None, None, 8, 8, 256, 1 << 20) == 2  # MISORT_ERR_NULL
    assert call(10, 256, None, None, None, 8, 8, 256, 1 << 20) == 2  # keys-only needs values_out
    assert call(10, 256, 512, None, None, 1 << 20, 1 << 20, 1 << 30, 16) == 4  # MISORT_ERR_SCRATCH
    assert "scratch too small" in lib.misort_last_error().decode()
    assert call(10, 258, 512, None, None, 8, 8, 1 << 20, 1 << 20) == 5  # MISORT_ERR_ALIGN
    assert call(10, 256, 512, None, None, 8, 8, (1 << 20) + 8, 1 << 20) == 5  # scratch alignment
    # argsort with values_out aliasing values_in
    assert call(10, 256, 256, None, 1024, 8, 8, 1 << 20, 1 << 20) == 7  # MISORT_ERR_ALIAS
    # scratch overlapping the input
    assert call(10, 1 << 20, (1 << 20) + 4096, None, None, 8, 8, 1 << 20, 1 << 20) == 7


def test_swap_last_argument_errors(lib):
    assert lib.misort_swap_last(None, None, 0, 0, 1, 0, 4, None) == 0
    assert lib.misort_swap_last(256, 512, 1, 4, 1, 4, 3, None) == 1
    assert lib.misort_swap_last(None, 512, 1, 4, 1, 4, 4, None) == 2


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmisort.so")
    with pytest.raises(_lib.MisortLibraryError):
        _lib.load()


def test_no_gpu_is_loud():
    import torch

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    import cunumeric_amd as num

    with pytest.raises(RuntimeError, match="needs a GPU"):
        num.sort([3, 1, 2])


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "cunumeric_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".sh")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f
