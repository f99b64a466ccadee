"""Long sorts of 8-byte keys run their radix passes over the upper five bytes first
(cunumeric_amd/csrc/upperfirst.hpp): a sample decides whether that is tried, one read of the
result sorts the short runs of keys that agree in those bytes, and the eight passes follow on
the device if a run was too long.  Through the C ABI with `upper_first` of misort_options (1:
any length; 2: tried whatever the sample says) on arrays small enough for numpy's stable sort
to check: inputs with no runs, short runs, runs at the limit of what the fix-up sorts, runs
beyond it (the way back), heavy ties, rows, payloads, float zeros and NaNs."""
import numpy as np
import pytest

from cunumeric_amd._lib import Options
from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu

TYPES = [np.int64, np.uint64, np.float64, np.complex64]


@pytest.fixture(scope="module")
def abi():
    return Abi()


def opts(mode):
    return Options(bucket_path=0, low_cardinality=0, upper_first=mode)


def from_keys(dtype, upper, low):
    """Elements of `dtype` whose sort keys have `upper` in their upper 40 bits and `low` in the
    lower 24 (positive floats, non-negative integers: the key order is the bit order)."""
    bits = (upper.astype(np.uint64) << np.uint64(24)) | low.astype(np.uint64)
    dt = np.dtype(dtype)
    if dt.kind == "f":
        return (bits & np.uint64(0x7FEFFFFFFFFFFFFF)).view(np.float64)   # finite, positive
    if dt.kind == "c":   # real part = upper 32 bits of the key, imaginary part below
        re = ((bits >> np.uint64(32)) & np.uint64(0x7F7FFFFF)).astype(np.uint32).view(np.float32)
        im = (bits & np.uint64(0x7F7FFFFF)).astype(np.uint32).view(np.float32)
        return (re + 1j * im).astype(np.complex64)
    return (bits >> np.uint64(1)).astype(dtype)   # (keeps int64 non-negative; the run structure stays)


def inputs(dtype, n, rng):
    out = {"random": random_array(dtype, n, rng)}
    full = rng.integers(0, 1 << 39, n)
    low = rng.integers(0, 1 << 24, n)
    out["no runs"] = from_keys(dtype, full, low)
    out["short runs"] = from_keys(dtype, rng.integers(0, n // 3, n) * 1000003, low)
    out["runs of 16 and 17"] = from_keys(dtype, np.repeat(rng.permutation(n // 16 + 1), 16)[:n] * 7919 +
                                         (np.arange(n) % 1000 == 0), low)
    out["long runs"] = from_keys(dtype, rng.integers(0, 500, n) * 100000007, low)
    out["heavy ties"] = out["random"][rng.integers(0, 100, n)]
    out["ties and runs"] = from_keys(dtype, rng.integers(0, n // 4, n) * 1000003, rng.integers(0, 3, n) << 20)
    # small values of both signs: every upper byte of an integer only repeats the sign, so the
    # passes over them are skipped or run over two values, and everything is left to the way back
    small = rng.integers(-1000, 1000, n)
    out["small, both signs"] = (small + 1j * rng.integers(-3, 3, n)).astype(dtype) if np.dtype(dtype).kind == "c" \
        else small.astype(dtype) if np.dtype(dtype) != np.uint64 else (small + 1000).astype(dtype)
    out["wide and small mixed"] = np.where(rng.integers(0, 2, n) == 0, out["small, both signs"], out["random"])
    return out


def check(abi, a, row_len, mode, **kw):
    rows = a.size // row_len
    a2 = a.reshape(rows, row_len)
    perm = np.argsort(a2, axis=1, kind="stable")
    got = abi.local_sort(a, row_len, argsort=True, options=opts(mode), **kw).reshape(rows, row_len)
    assert np.array_equal(got, perm)
    vals = abi.local_sort(a, row_len, argsort=False, options=opts(mode)).reshape(rows, row_len)
    assert bits_equal(vals, np.take_along_axis(a2, perm, axis=1))


@pytest.mark.parametrize("dtype", TYPES, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("mode", [1, 2], ids=["sample decides", "always tried"])
def test_every_kind_of_run(abi, dtype, mode):
    rng = np.random.default_rng(91)
    n = 300007
    plan = abi.describe_plan(dtype, n, n, True, options=opts(mode))
    assert f"upper_first_attempt={mode}" in plan, plan
    for name, a in inputs(dtype, n, rng).items():
        print(f"upper first dtype={np.dtype(dtype).name} mode={mode} case={name}", flush=True)
        check(abi, a, n, mode)


@pytest.mark.parametrize("dtype", TYPES, ids=lambda d: np.dtype(d).name)
def test_rows_payloads_and_in_place(abi, dtype):
    rng = np.random.default_rng(92)
    rows, row_len = 3, 100003
    for name in ("random", "short runs", "long runs"):
        a = np.concatenate([inputs(dtype, row_len, rng)[name] for _ in range(rows)])
        print(f"upper first rows dtype={np.dtype(dtype).name} case={name}", flush=True)
        for mode in (1, 2):
            check(abi, a, row_len, mode)
        perm = np.argsort(a.reshape(rows, row_len), axis=1, kind="stable")
        pay = rng.integers(-2**62, 2**62, a.size, dtype=np.int64)
        want = np.take_along_axis(pay.reshape(rows, row_len), perm, axis=1)
        for inplace in (False, True):   # (in place the attempt is not made: the way back needs the input)
            got = abi.local_sort(a, row_len, argsort=True, indices_in=pay, inplace=inplace, options=opts(2))
            assert np.array_equal(got.reshape(rows, row_len), want)
        assert np.array_equal(abi.local_sort(a, row_len, argsort=True, index_offset=11, options=opts(2)).reshape(rows, -1),
                              perm + 11)
        got = abi.local_sort(a, row_len, argsort=False, inplace=True, options=opts(2)).reshape(rows, row_len)
        assert bits_equal(got, np.take_along_axis(a.reshape(rows, row_len), perm, axis=1))
        if np.dtype(dtype).kind != "c":
            idx, vals = abi.local_sort(a, row_len, argsort=True, want_values=True, options=opts(2))
            assert np.array_equal(idx.reshape(rows, row_len), perm)
            assert bits_equal(vals.reshape(rows, row_len), np.take_along_axis(a.reshape(rows, row_len), perm, axis=1))


def test_float_zeros_and_nans_keep_their_bits(abi):
    rng = np.random.default_rng(93)
    n = 250001
    a = rng.standard_normal(n)
    a[rng.integers(0, n, 2000)] = 0.0
    a[rng.integers(0, n, 2000)] = -0.0
    a[rng.integers(0, n, 500)] = np.nan
    a[rng.integers(0, n, 500)] = np.float64(np.uint64(0xFFF8000000000123).view(np.float64))
    a[rng.integers(0, n, 50)] = np.inf
    a[rng.integers(0, n, 50)] = -np.inf
    for mode in (1, 2):
        check(abi, a, n, mode)
    c = np.empty(n // 2, dtype=np.complex64)
    c.real = a[: n // 2]
    c.imag = a[n // 2: 2 * (n // 2)]
    for mode in (1, 2):
        check(abi, c, c.size, mode)


def test_runs_at_the_ends_of_rows_and_of_the_fix_up_stretches(abi):
    """Runs of equal upper bits placed across the boundaries between the fix-up's stretches of
    4096 elements and at both ends of every row."""
    rng = np.random.default_rng(94)
    rows, row_len = 4, 40000
    upper = np.sort(rng.integers(0, 1 << 30, (rows, row_len)), axis=1) * 300
    for r in range(rows):
        for start in (0, 4090, 8185, 12283, row_len - 9, row_len - 16):
            upper[r, start:start + rng.integers(2, 16)] = upper[r, start]
    low = rng.integers(0, 1 << 24, rows * row_len)
    shuffle = np.argsort(rng.random((rows, row_len)), axis=1)
    for dtype in (np.int64, np.float64):
        a = from_keys(dtype, np.take_along_axis(upper, shuffle, axis=1).reshape(-1), low)
        check(abi, a, row_len, 2)


def test_built_in_choice_starts_at_two_to_the_25(abi):
    assert "upper_first_attempt=1" in abi.describe_plan(np.float64, 1 << 25, 1 << 25, True)
    assert "upper_first_attempt" not in abi.describe_plan(np.float64, (1 << 25) - 1, (1 << 25) - 1, True)
    assert "upper_first_attempt" not in abi.describe_plan(np.float32, 1 << 26, 1 << 26, True)
    assert "upper_first_attempt" not in abi.describe_plan(np.complex128, 1 << 25, 1 << 25, True)
    assert "upper_first_attempt" not in abi.describe_plan(np.int64, 1 << 26, 1 << 26, True, options=Options(upper_first=0))


@pytest.mark.parametrize("dtype", [np.int64, np.float64, np.complex64], ids=lambda d: np.dtype(d).name)
def test_two_to_the_25_elements_with_the_built_in_choice(abi, dtype):
    """The size from which the attempt is made by itself: uniform keys (a handful of pairs agree
    in their upper bits), against numpy's stable sort."""
    rng = np.random.default_rng(95)
    n = 1 << 25
    if np.dtype(dtype).kind == "i":
        a = rng.integers(-2**63, 2**63 - 1, n, dtype=np.int64)
    elif np.dtype(dtype).kind == "f":
        a = rng.standard_normal(n)
    else:
        a = (rng.standard_normal(n, dtype=np.float32) + 1j * rng.standard_normal(n, dtype=np.float32)).astype(np.complex64)
    assert "upper_first_attempt=1" in abi.describe_plan(dtype, n, n, True)
    print(f"upper first 2^25 dtype={np.dtype(dtype).name}", flush=True)
    assert np.array_equal(abi.local_sort(a, n, argsort=True), np.argsort(a, kind="stable"))
    assert bits_equal(abi.local_sort(a, n, argsort=False), np.sort(a, kind="stable"))


@pytest.mark.parametrize("seed", range(12))
def test_random_run_structures(abi, seed):
    """Random lengths, rows, run-length distributions (means from 1 to 12: some runs beyond what
    the fix-up sorts, so both outcomes of the attempt occur), ties inside runs, every 8-byte type."""
    rng = np.random.default_rng(1000 + seed)
    dtype = TYPES[seed % len(TYPES)]
    rows = int(rng.integers(1, 4))
    row_len = int(rng.integers(16385, 150000))
    n = rows * row_len
    mean = float(rng.choice([1.0, 1.5, 3.0, 6.0, 12.0]))
    lengths = rng.geometric(1.0 / mean, n)
    upper = np.repeat(rng.permutation(lengths.size), lengths)[:n] * int(rng.integers(1, 5000))
    low = rng.integers(0, 1 << int(rng.integers(1, 33)), n)   # (few low bits: ties inside the runs)
    a = from_keys(dtype, upper[rng.permutation(n)], low)
    print(f"upper first random seed={seed} dtype={np.dtype(dtype).name} rows={rows} row_len={row_len} mean run={mean}",
          flush=True)
    check(abi, a, row_len, 2)
    check(abi, a, row_len, 1)
