"""Radix passes over a digit that is the same in every key are skipped on the device (the
first upsweep ORs the keys and their complements; every later kernel derives from those
words which passes are dead and which ping-pong buffer holds its input).  Large sorts also
leave out the passes over the most significant digits if those are constant: the last pass
whose digit varies then writes the result; early_last_min_bytes = 0 in the options of
misort_local_opts makes small sorts do the same, which is how the tests below reach that path
(they also ask for the radix path, which single rows of this length no longer take by themselves).  Inputs whose
constant bytes sit in every combination of positions, for all key widths with middle passes,
sorts and argsorts, rows, a caller payload, and the same input with the skipping switched
off must agree with NumPy."""
import os
import subprocess
import sys

import numpy as np
import pytest

from tests.util import Abi, bits_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    a = Abi()
    a.force_radix = True
    return a


@pytest.fixture(params=[False, True], ids=["top pass kept", "last live pass writes the result"])
def early_last(request, abi):
    abi.early_last_bytes = 0 if request.param else 1 << 40
    yield request.param
    abi.early_last_bytes = None


def masked_random(dtype, n, rng, live_bytes):
    """Unsigned random values in which only the bytes listed in live_bytes vary; the others
    carry a fixed non-zero pattern."""
    dt = np.dtype(dtype)
    u = np.dtype(f"u{dt.itemsize}")
    x = rng.integers(0, np.iinfo(u).max, n, dtype=u, endpoint=True)
    mask = sum(0xFF << (8 * b) for b in live_bytes)
    const = rng.integers(0, np.iinfo(u).max, dtype=u, endpoint=True)
    x = (x & u.type(mask)) | (const & u.type(~mask & np.iinfo(u).max))
    return x.view(dt) if dt.kind != "u" else x


WIDTH4 = [(0,), (0, 1), (0, 3), (1, 2), (3,), (0, 1, 2, 3), (), (2,)]
WIDTH8 = [(0,), (0, 1), (0, 7), (3, 4), (7,), (1, 2, 3, 4, 5, 6), (0, 2, 4, 6), (), (0, 1, 2, 3, 4, 5, 6, 7), (5,)]


@pytest.mark.parametrize("dtype,patterns", [(np.uint32, WIDTH4), (np.int32, WIDTH4), (np.uint64, WIDTH8),
                                             (np.int64, WIDTH8)], ids=["uint32", "int32", "uint64", "int64"])
def test_constant_bytes_in_every_position(abi, dtype, patterns, early_last):
    rng = np.random.default_rng(61)
    n = 300007
    if os.environ.get("MISORT_SKIP_PASSES") != "0":
        assert ("early_last=1" in abi.describe_plan(dtype, n, n, True)) == early_last
    for live in patterns:
        a = masked_random(dtype, n, rng, live)
        for chunks in (0, 3):
            print(f"skip passes dtype={np.dtype(dtype).name} live bytes={live} chunks={chunks}", flush=True)
            assert np.array_equal(abi.local_sort(a, n, argsort=False, chunks=chunks), np.sort(a, kind="stable")), live
            assert np.array_equal(abi.local_sort(a, n, argsort=True, chunks=chunks), np.argsort(a, kind="stable")), live


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64, np.complex64, np.complex128],
                         ids=lambda d: np.dtype(d).name)
def test_small_ranges_rows_and_payload(abi, dtype, early_last):
    """Values from a small range (the usual case for integer data): the upper digits of the
    keys are constant.  Floats and complex numbers built from small integers have constant
    low mantissa bytes instead."""
    rng = np.random.default_rng(62)
    rows, row_len = 3, 120001
    a = rng.integers(0, 1000, rows * row_len).astype(dtype).reshape(rows, row_len)
    if np.dtype(dtype).kind == "c":
        a = a + 1j * rng.integers(0, 50, a.shape).astype(a.real.dtype)
    print(f"skip passes small range dtype={np.dtype(dtype).name}", flush=True)
    got = abi.local_sort(a, row_len, argsort=True, chunks=2 * rows).reshape(rows, row_len)
    assert np.array_equal(got, np.argsort(a, axis=1, kind="stable"))
    got = abi.local_sort(a, row_len, argsort=False).reshape(rows, row_len)
    assert bits_equal(got, np.sort(a, axis=1, kind="stable"))
    pay = rng.integers(-(2**62), 2**62, rows * row_len, dtype=np.int64)
    got = abi.local_sort(a, row_len, argsort=True, indices_in=pay).reshape(rows, row_len)
    ref = np.take_along_axis(pay.reshape(rows, row_len), np.argsort(a, axis=1, kind="stable"), axis=1)
    assert np.array_equal(got, ref)
    # in place
    flat = a.reshape(-1).copy()
    got = abi.local_sort(flat[:row_len], row_len, argsort=False, inplace=True)
    assert bits_equal(got, np.sort(flat[:row_len], kind="stable"))


@pytest.mark.parametrize("dtype", [np.int32, np.int64], ids=lambda d: np.dtype(d).name)
def test_small_values_of_both_signs(abi, dtype, early_last):
    """Signed integers near zero: the upper bytes only repeat the sign (0x00 / 0xFF), which
    the pass over the most significant byte sorts out, so the passes over them are left out
    although their digits differ between keys."""
    rng = np.random.default_rng(65)
    ii = np.iinfo(dtype)
    n = 250007
    ranges = [(-1000, 1000), (-70000, 5), (-1, 0), (-50000, -1), (-3, 300), (ii.min, ii.min + 1000),
              (ii.max - 5, ii.max), (-(1 << (ii.bits - 9)), 1 << (ii.bits - 9))]
    for lo, hi in ranges:
        a = rng.integers(lo, hi, n, dtype=dtype, endpoint=True)
        print(f"skip passes signed dtype={np.dtype(dtype).name} range=({lo}, {hi})", flush=True)
        assert np.array_equal(abi.local_sort(a, n, argsort=False), np.sort(a)), (lo, hi)
        assert np.array_equal(abi.local_sort(a, n, argsort=True, chunks=5), np.argsort(a, kind="stable")), (lo, hi)
    # a few far-off values among small ones, rows, and the extremes
    a = rng.integers(-500, 500, 3 * 100003, dtype=dtype)
    a[rng.integers(0, a.size, 7)] = [ii.min, ii.max, ii.min + 1, -1, 0, ii.max - 1, 1 << (ii.bits - 2)]
    a = a.reshape(3, 100003)
    got = abi.local_sort(a, 100003, argsort=True).reshape(3, -1)
    assert np.array_equal(got, np.argsort(a, axis=1, kind="stable"))
    assert np.array_equal(abi.local_sort(a, 100003, argsort=False).reshape(3, -1), np.sort(a, axis=1))


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=lambda d: np.dtype(d).name)
def test_float_values_with_constant_mantissa_bytes(abi, dtype, early_last):
    """Keys-only float sorts out of place: integer-valued floats have constant low mantissa
    bytes, whose passes are skipped; the zeros of both signs and the NaNs (with their
    payloads) are restored from the input after the sort.  In place every pass runs (the
    zeros and NaNs are set aside before the last one); both must give NumPy's bits."""
    rng = np.random.default_rng(66)
    rows, n = 2, 150001
    for hi in (200, 60000, 1 << 22):
        a = rng.integers(-hi, hi, rows * n).astype(dtype)
        u = a.view(np.dtype(f"u{a.dtype.itemsize}"))
        where = rng.integers(0, a.size, a.size // 50)
        a[where[: where.size // 3]] = -0.0
        a[where[where.size // 3: 2 * where.size // 3]] = 0.0
        nan_bits = (np.array(np.nan, dtype=dtype).view(u.dtype) | rng.integers(1, 1000, where.size).astype(u.dtype))
        u[where[2 * where.size // 3:]] = nan_bits[2 * where.size // 3:]
        a = a.reshape(rows, n)
        ref = np.sort(a, axis=1, kind="stable")
        print(f"skip passes float values dtype={np.dtype(dtype).name} below {hi}", flush=True)
        got = abi.local_sort(a, n, argsort=False).reshape(rows, n)
        assert bits_equal(got, ref), hi
        got = abi.local_sort(a, n, argsort=False, chunks=7).reshape(rows, n)
        assert bits_equal(got, ref), hi
        got = abi.local_sort(a, n, argsort=False, inplace=True).reshape(rows, n)
        assert bits_equal(got, ref), hi


def test_large_int64_small_range(abi, early_last):
    rng = np.random.default_rng(63)
    n = 1 << 24
    a = rng.integers(0, 50000, n, dtype=np.int64)
    print("skip passes int64 2^24 values below 50000", flush=True)
    assert np.array_equal(abi.local_sort(a, n, argsort=True), np.argsort(a, kind="stable"))
    assert np.array_equal(abi.local_sort(a, n, argsort=False), np.sort(a))
    if os.environ.get("MISORT_SKIP_PASSES") != "0":
        assert "skip_dead_passes=1" in abi.describe_plan(np.int64, n, n, True)


def test_switch_off_gives_the_same_result():
    code = (
        "import numpy as np, sys\n"
        "from tests.util import Abi\n"
        "rng = np.random.default_rng(64)\n"
        "a = rng.integers(0, 300, 400001, dtype=np.int64)\n"
        "abi = Abi()\n"
        "abi.force_radix = True\n"
        "plan = abi.describe_plan(np.int64, a.size, a.size, True)\n"
        "s = abi.local_sort(a, a.size, argsort=True, chunks=3)\n"
        "sys.stdout.write(plan + '\\n' + str(bool((s == np.argsort(a, kind='stable')).all())) + '\\n')\n"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    outs = []
    for flag in ("1", "0"):
        env = dict(os.environ, MISORT_SKIP_PASSES=flag, PYTHONPATH=root)
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=root,
                           timeout=240)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append(r.stdout.strip().splitlines())
    assert outs[0][-1] == "True" and outs[1][-1] == "True"
    assert "skip_dead_passes=1" in outs[0][0] and "skip_dead_passes" not in outs[1][0]
