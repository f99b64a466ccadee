"""Keys-only radix sorts of 8-byte elements write a digit side-band (the next pass's digit
of every key as one byte, in whole 128-byte lines through a byte carry) that the next
upsweep counts instead of the keys.  Chunks long enough that lines complete many times,
heavy digit values (runs longer than a line per tile), rows whose starts are not multiples
of 128 elements, and the sort with the side-band switched off must all agree with NumPy."""
import os
import subprocess
import sys

import numpy as np
import pytest

from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    a = Abi()
    a.force_radix = True  # (single rows of this length would take the four-launch path otherwise)
    return a


def cases(dtype, n, rng):
    dt = np.dtype(dtype)
    out = {"random": random_array(dtype, n, rng), "narrow": random_array(dtype, n, rng, narrow=True)}
    if dt.kind in "iu":
        ii = np.iinfo(dt)
        vals = rng.integers(ii.min, ii.max, 16, dtype=dt, endpoint=True)
        w = np.arange(1, 17, dtype=np.float64) ** -1.2
        out["16 values"] = vals[rng.choice(16, n, p=w / w.sum())]
        out["small range"] = rng.integers(0, 1000, n).astype(dt)     # upper digits constant
        out["sorted"] = np.sort(out["random"])
        out["reversed"] = out["sorted"][::-1].copy()
    else:
        out["unit interval"] = rng.random(n).astype(dt)
        out["constant"] = np.full(n, 1.5, dtype=dt)
    return out


@pytest.mark.parametrize("dtype", [np.int64, np.uint64, np.float64], ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("chunks", [1, 4, 0], ids=["one chunk", "four chunks", "default plan"])
def test_long_chunks(abi, dtype, chunks):
    rng = np.random.default_rng(41)
    n = (1 << 21) + 777
    for name, a in cases(dtype, n, rng).items():
        print(f"side-band dtype={np.dtype(dtype).name} chunks={chunks} case={name}", flush=True)
        got = abi.local_sort(a, n, argsort=False, chunks=chunks)
        assert bits_equal(got, np.sort(a, kind="stable")), name


@pytest.mark.parametrize("dtype", [np.int64, np.float64], ids=lambda d: np.dtype(d).name)
def test_rows_with_unaligned_starts(abi, dtype):
    rng = np.random.default_rng(42)
    rows, row_len = 5, 100003          # row starts at odd offsets: first and last lines are partial
    a = random_array(dtype, rows * row_len, rng).reshape(rows, row_len)
    for chunks in (rows, 3 * rows):
        print(f"side-band rows dtype={np.dtype(dtype).name} chunks={chunks}", flush=True)
        got = abi.local_sort(a, row_len, argsort=False, chunks=chunks).reshape(rows, row_len)
        assert bits_equal(got, np.sort(a, axis=1, kind="stable"))


def test_in_place_and_large(abi):
    rng = np.random.default_rng(43)
    n = 1 << 25
    a = rng.integers(-(2**63), 2**63, n, dtype=np.int64)
    print("side-band int64 2^25 default plan", flush=True)
    assert np.array_equal(abi.local_sort(a, n, argsort=False), np.sort(a))
    print("side-band int64 2^25 in place", flush=True)
    assert np.array_equal(abi.local_sort(a, n, argsort=False, inplace=True), np.sort(a))


def test_switch_off_gives_the_same_result():
    """MISORT_SIDE_BAND=0 (read when the library is first used) sorts without the side-band:
    a fresh process, same input, same bytes out."""
    code = (
        "import numpy as np, sys\n"
        "from tests.util import Abi\n"
        "rng = np.random.default_rng(44)\n"
        "a = rng.standard_normal(300001)\n"
        "abi = Abi()\n"
        "abi.force_radix = True\n"
        "plan = abi.describe_plan(np.float64, a.size, a.size, False)\n"
        "s = abi.local_sort(a, a.size, argsort=False, chunks=3)\n"
        "sys.stdout.write(plan + '\\n' + str(bool((s == np.sort(a)).all())) + '\\n')\n"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    outs = []
    for flag in ("1", "0"):
        env = dict(os.environ, MISORT_SIDE_BAND=flag, PYTHONPATH=root)
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=root,
                           timeout=240)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append(r.stdout.strip().splitlines())
    assert outs[0][-1] == "True" and outs[1][-1] == "True"
    assert "side_band=1" in outs[0][0] and "side_band=0" in outs[1][0]


# ---- sorts with positions (and 16-byte keys): a pass writes the side-band, without the byte
# carry, only for rows in which few digit values are in use, and says so per row ----

def few_values(dtype, n, rng, k=16):
    dt = np.dtype(dtype)
    if dt.kind in "iu":
        ii = np.iinfo(dt)
        vals = rng.integers(ii.min, ii.max, k, dtype=dt, endpoint=True)
    elif dt.kind == "c":
        vals = (rng.standard_normal(k) + 1j * rng.standard_normal(k)).astype(dt)
    else:
        vals = rng.standard_normal(k).astype(dt)
    w = np.arange(1, k + 1, dtype=np.float64) ** -1.2
    return vals[rng.choice(k, n, p=w / w.sum())]


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64, np.float64, np.complex64, np.complex128],
                         ids=lambda d: np.dtype(d).name)
def test_argsort_few_digit_values(abi, dtype):
    rng = np.random.default_rng(51)
    n = (1 << 20) + 4321
    inputs = {"16 values": few_values(dtype, n, rng), "3 values": few_values(dtype, n, rng, 3)}
    if np.dtype(dtype).kind in "iu":
        inputs["small range"] = rng.integers(0, 200, n).astype(dtype)   # upper digits all equal
    for name, a in inputs.items():
        for chunks in (0, 5):
            print(f"adaptive side-band dtype={np.dtype(dtype).name} case={name} chunks={chunks}", flush=True)
            got = abi.local_sort(a, n, argsort=True, chunks=chunks)
            assert np.array_equal(got, np.argsort(a, kind="stable")), (name, chunks)
    if np.dtype(dtype).kind == "c":   # 16-byte keys (complex128) and complex64 also sort values through positions
        a = inputs["16 values"]
        assert bits_equal(abi.local_sort(a, n, argsort=False), np.sort(a, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float64], ids=lambda d: np.dtype(d).name)
def test_rows_that_decide_differently(abi, dtype):
    """Rows with few values, a constant row and random rows in one call: every row decides
    for itself in every pass, and the next upsweep must follow each row's own flag."""
    rng = np.random.default_rng(52)
    rows, row_len = 6, 150001
    a = np.empty((rows, row_len), dtype=dtype)
    a[0] = few_values(dtype, row_len, rng)
    a[1] = random_array(dtype, row_len, rng)
    a[2] = np.full(row_len, a[1, 0], dtype=dtype)
    a[3] = random_array(dtype, row_len, rng, narrow=True)
    a[4] = random_array(dtype, row_len, rng)
    a[5] = few_values(dtype, row_len, rng, 40)
    for chunks in (rows, 4 * rows):
        print(f"adaptive side-band rows dtype={np.dtype(dtype).name} chunks={chunks}", flush=True)
        got = abi.local_sort(a, row_len, argsort=True, chunks=chunks).reshape(rows, row_len)
        assert np.array_equal(got, np.argsort(a, axis=1, kind="stable"))
    pay = rng.integers(-(2**62), 2**62, rows * row_len, dtype=np.int64)
    got = abi.local_sort(a, row_len, argsort=True, indices_in=pay, chunks=2 * rows).reshape(rows, row_len)
    ref = np.take_along_axis(pay.reshape(rows, row_len), np.argsort(a, axis=1, kind="stable"), axis=1)
    assert np.array_equal(got, ref)
