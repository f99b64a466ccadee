"""Randomly drawn calls of misort_local through the C ABI, each checked against NumPy: values out
of place and in place, positions with an offset, a caller's payload, positions together with
values, chunk targets that make small arrays walk several tiles, the entry point with the
library's own scratch, and the early last pass forced on and off; all 14 element types, rows
from one element to several hundred thousand, full-range, tied, repeated and small-range
values."""
import numpy as np
import pytest

from tests.util import ALL_DTYPES, Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu

ROW_LENGTHS = [1, 5, 33, 64, 200, 1024, 1025, 3000, 4096, 8192, 8193, 16384, 16385, 40000, 65536, 70001,
               150000, 400000]


@pytest.fixture(scope="module", params=[False, True], ids=["default plan", "radix path asked for"])
def abi(request):
    # single rows of 16385 to about a million elements take the four-launch path by default;
    # the second round runs the same cases on the radix path, which serves the longer rows
    a = Abi()
    a.force_radix = request.param
    return a


def draw(rng, dtype, total, kind):
    if kind == 0:
        return random_array(dtype, total, rng)
    if kind == 1:
        return random_array(dtype, total, rng, narrow=True)
    if kind == 2:
        pool = random_array(dtype, max(2, total // int(rng.choice([4, 64, 1024]))), rng)
        return pool[rng.integers(0, pool.size, total)]
    if np.dtype(dtype).kind in "iu":
        r = int(rng.choice([3, 300, 70000]))
        a = rng.integers(-r if np.dtype(dtype).kind == "i" else 0, r, total)
        return np.clip(a, np.iinfo(dtype).min, np.iinfo(dtype).max).astype(dtype)
    return random_array(dtype, total, rng, specials=False)


def same_bits_or_values(got, ref):
    return bits_equal(got, ref) or np.array_equal(got, ref, equal_nan=True)


@pytest.mark.parametrize("seed", range(4))
def test_random_calls(abi, seed):
    rng = np.random.default_rng(2000 + seed)
    for it in range(150):
        dtype = ALL_DTYPES[rng.integers(0, len(ALL_DTYPES))]
        row = int(rng.choice(ROW_LENGTHS))
        rows = max(1, min(int(rng.choice([1, 1, 2, 7, 50])), 1_200_000 // row))
        a = draw(rng, dtype, rows * row, int(rng.integers(0, 4))).reshape(rows, row)
        mode = int(rng.integers(0, 6))
        static = bool(rng.integers(0, 5) == 0) and a.nbytes < (4 << 20)
        chunks = 0 if static else int(rng.choice([0, 0, 1, 3, 16, 1000]))
        off = int(rng.choice([0, 0, 17, -5, 1 << 40]))
        tag = (f"seed={seed} it={it} dtype={np.dtype(dtype).name} rows={rows} row={row} mode={mode} "
               f"chunks={chunks} static={static} off={off}")
        print(tag, flush=True)
        s = np.sort(a, axis=1, kind="stable")
        perm = np.argsort(a, axis=1, kind="stable")
        kw = dict(chunks=chunks, static=static)
        if mode == 0:    # values, out of place
            assert same_bits_or_values(abi.local_sort(a, row, argsort=False, **kw).reshape(rows, row), s), tag
        elif mode == 1:  # values, in place
            got = abi.local_sort(a, row, argsort=False, inplace=True, **kw).reshape(rows, row)
            assert same_bits_or_values(got, s), tag
        elif mode == 2:  # positions with an offset
            got = abi.local_sort(a, row, argsort=True, index_offset=off, **kw).reshape(rows, row)
            assert np.array_equal(got, perm + off), tag
        elif mode == 3:  # a caller's payload, out of place or in place
            pay = rng.integers(-(2**62), 2**62, rows * row, dtype=np.int64)
            got = abi.local_sort(a, row, argsort=True, indices_in=pay, inplace=bool(rng.integers(0, 2)), **kw)
            assert np.array_equal(got.reshape(rows, row), np.take_along_axis(pay.reshape(rows, row), perm, axis=1)), tag
        elif mode == 4:  # positions and values
            gi, gv = abi.local_sort(a, row, argsort=True, want_values=True, index_offset=off, **kw)
            assert np.array_equal(gi.reshape(rows, row), perm + off), tag
            assert same_bits_or_values(gv.reshape(rows, row), s), tag
        else:            # the early last pass on for every size, or for none
            if static:
                kw = dict(chunks=chunks)
            got = abi.local_sort(a, row, argsort=True, early_last_bytes=int(rng.choice([0, 1 << 40])),
                                 **kw).reshape(rows, row)
            assert np.array_equal(got, perm), tag
