"""The four-launch sort of single rows of a few ten thousand to a million elements (sample
splitters -> count -> scatter into bins -> radix sort of every bin inside one workgroup;
cunumeric_amd/csrc/bucket.hpp), through the C ABI, bit-exact against numpy's stable sort and
the oracle: every dtype it serves, keys only and with positions, caller payloads, in place,
heavy ties (bins of equal keys), inputs that defeat evenly spaced sampling, bins too long for
the registers (forced through the options of misort_local_opts) and the ballot ranking."""
import os
import subprocess
import sys

import numpy as np
import pytest

from cunumeric_amd._lib import Options
from oracle import misort_oracle as oracle
from tests.util import ALL_DTYPES, Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SERVED = [d for d in ALL_DTYPES if np.dtype(d) != np.complex128]


@pytest.fixture(scope="module")
def abi():
    return Abi()


def check(abi, a, **kw):
    n = a.size
    idx = abi.local_sort(a, n, argsort=True, **kw)
    assert np.array_equal(idx, np.argsort(a, kind="stable"))
    vals = abi.local_sort(a, n, argsort=False, **kw)
    assert bits_equal(vals, np.sort(a, kind="stable"))


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
def test_every_dtype_over_the_sizes_the_path_serves(abi, dtype):
    rng = np.random.default_rng(71)
    for n in (16385, 20001, (1 << 15) + 3, 1 << 16, 100003, 1 << 18):
        for narrow in (False, True):
            a = random_array(dtype, n, rng, narrow=narrow)
            print(f"bucket dtype={np.dtype(dtype).name} n={n} narrow={narrow}", flush=True)
            # (1-byte keys never take the path by themselves, one radix pass being quicker,
            # and 2-byte keys with positions up to 2^18 elements only: asked for here)
            kw = dict(options=Options(bucket_path=1)) if np.dtype(dtype).itemsize <= 2 else {}
            plan = abi.describe_plan(dtype, n, n, True, **kw)
            if np.dtype(dtype) != np.complex128:
                assert "strategy=bucket" in plan, plan
            check(abi, a, **kw)
            assert np.array_equal(abi.local_sort(a, n, argsort=True, **kw), oracle.local_sort(a, n, True))


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.uint64, np.float64, np.complex64],
                         ids=lambda d: np.dtype(d).name)
def test_a_million_elements(abi, dtype):
    rng = np.random.default_rng(72)
    for n in (1 << 19, (1 << 20) - 7, 1 << 20):
        a = random_array(dtype, n, rng)
        print(f"bucket dtype={np.dtype(dtype).name} n={n} plan={abi.describe_plan(dtype, n, n, True)}", flush=True)
        check(abi, a)


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32, np.float32, np.int64, np.float64, np.complex64],
                         ids=lambda d: np.dtype(d).name)
def test_payload_in_place_offset_and_values(abi, dtype):
    rng = np.random.default_rng(73)
    n = 70001
    kw = dict(options=Options(bucket_path=1)) if np.dtype(dtype).itemsize == 1 else {}
    a = random_array(dtype, n, rng)
    ref = np.argsort(a, kind="stable")
    pay = rng.integers(-2**62, 2**62, n, dtype=np.int64)
    for inplace in (False, True):
        got = abi.local_sort(a, n, argsort=True, indices_in=pay, inplace=inplace, **kw)
        assert np.array_equal(got, pay[ref])
    assert np.array_equal(abi.local_sort(a, n, argsort=True, index_offset=12345, **kw), ref + 12345)
    assert bits_equal(abi.local_sort(a, n, argsort=False, inplace=True, **kw), np.sort(a, kind="stable"))
    idx, vals = abi.local_sort(a, n, argsort=True, want_values=True, **kw)
    assert np.array_equal(idx, ref) and bits_equal(vals, a[ref])
    if np.dtype(dtype).kind != "c":
        idx, vals = abi.local_sort(a, n, argsort=True, indices_in=pay, want_values=True, **kw)
        assert np.array_equal(idx, pay[ref]) and bits_equal(vals, a[ref])


@pytest.mark.parametrize("dtype", SERVED, ids=lambda d: np.dtype(d).name)
def test_several_rows_side_by_side(abi, dtype):
    """Rows too long for the row kernels whose total stays within the path's length: every row
    gets its own splitters, counts and bins (second launch dimension).  Rows that differ in
    kind (random, constant, few values, sorted), row starts that are not multiples of a line,
    a caller's payload, in place, an index offset."""
    rng = np.random.default_rng(77)
    for rows, row_len in ((3, 20001), (7, 40003), (2, 300001), (30, 17001)):
        a = random_array(dtype, rows * row_len, rng).reshape(rows, row_len)
        a[0] = a[0, 0]
        if rows > 2:
            a[1] = a[1, rng.integers(0, 5, row_len)]
            a[2] = np.sort(a[2], kind="stable")
        kw = dict(options=Options(bucket_path=1))   # (where the path ends by itself depends on the type)
        plan = abi.describe_plan(dtype, a.size, row_len, True, **kw)
        print(f"bucket rows dtype={np.dtype(dtype).name} rows={rows} row_len={row_len} plan={plan}", flush=True)
        assert "strategy=bucket" in plan, plan
        perm = np.argsort(a, axis=1, kind="stable")
        got = abi.local_sort(a, row_len, argsort=True, **kw).reshape(rows, row_len)
        assert np.array_equal(got, perm)
        vals = abi.local_sort(a, row_len, argsort=False, **kw).reshape(rows, row_len)
        assert bits_equal(vals, np.take_along_axis(a, perm, axis=1))
        assert bits_equal(abi.local_sort(a, row_len, argsort=False, inplace=True, **kw).reshape(rows, row_len),
                          np.take_along_axis(a, perm, axis=1))
        assert np.array_equal(abi.local_sort(a, row_len, argsort=True, index_offset=7, **kw).reshape(rows, row_len),
                              perm + 7)
        pay = rng.integers(-2**62, 2**62, a.size, dtype=np.int64)
        want = np.take_along_axis(pay.reshape(rows, row_len), perm, axis=1)
        for inplace in (False, True):
            got = abi.local_sort(a, row_len, argsort=True, indices_in=pay, inplace=inplace, **kw).reshape(rows, row_len)
            assert np.array_equal(got, want)
        assert np.array_equal(abi.local_sort(a, row_len, argsort=True, **kw),
                              oracle.local_sort(a.reshape(-1), row_len, True))


def test_where_the_path_ends_by_itself(abi):
    """The built-in limits: measured against the radix passes per element size."""
    bucket = lambda dtype, vol, row, arg: "strategy=bucket" in abi.describe_plan(dtype, vol, row, arg)
    assert bucket(np.int32, 1 << 21, 1 << 21, False) and bucket(np.int32, 1 << 21, 1 << 21, True)
    assert not bucket(np.int32, (1 << 21) + 1, (1 << 21) + 1, False)
    assert bucket(np.int32, 3 << 19, 3 << 16, False) and not bucket(np.int32, 1 << 21, 1 << 18, False)
    assert bucket(np.float64, 1 << 21, 1 << 21, False) and bucket(np.float64, 1 << 21, 1 << 21, True)
    assert not bucket(np.float64, (1 << 21) + 1, (1 << 21) + 1, True)
    assert bucket(np.int64, 1 << 22, 1 << 19, True) and not bucket(np.int64, 1 << 23, 1 << 19, True)
    assert bucket(np.int16, 1 << 19, 1 << 19, False) and not bucket(np.int16, 1 << 20, 1 << 20, False)
    assert bucket(np.float16, 1 << 20, 1 << 20, False)
    assert bucket(np.int16, 1 << 18, 1 << 18, True) and not bucket(np.int16, 1 << 19, 1 << 19, True)
    assert not bucket(np.int8, 1 << 16, 1 << 16, True) and not bucket(np.uint8, 1 << 17, 1 << 15, False)
    assert not bucket(np.complex128, 1 << 16, 1 << 16, True)
    assert "strategy=radix" in abi.describe_plan(np.int32, 64 << 20, 1 << 20, True)


def adversarial(kind, n, rng):
    if kind == "sorted":
        return np.sort(rng.integers(-2**31, 2**31, n, dtype=np.int64)).astype(np.int32)
    if kind == "reversed":
        return np.sort(rng.standard_normal(n).astype(np.float32))[::-1].copy()
    if kind == "constant":
        return np.full(n, -7, dtype=np.int64)
    if kind == "two_values":
        return rng.integers(0, 2, n).astype(np.float64) * 3.5 - 1.0
    if kind == "sawtooth":
        return ((np.arange(n) % 3126) * 1000003 % (2**31)).astype(np.int32)
    if kind == "zipf16":
        v = rng.integers(-2**63, 2**63, 16, dtype=np.int64)
        w = np.arange(1, 17, dtype=np.float64) ** -1.2
        return v[rng.choice(16, n, p=w / w.sum())]
    if kind == "all_nan_and_zeros":
        a = np.where(rng.random(n) < 0.5, np.float32(np.nan), np.float32(0.0))
        a[rng.integers(0, n, n // 7)] = -0.0
        b = a.view(np.uint32).copy()
        nan = np.isnan(a)
        b[nan] |= rng.integers(1, 2**22, int(nan.sum()), dtype=np.uint32)
        b[nan] ^= rng.integers(0, 2, int(nan.sum()), dtype=np.uint32) << np.uint32(31)
        return b.view(np.float32)
    if kind == "lognormal":
        return np.exp(rng.standard_normal(n) * 9).astype(np.float32)
    if kind == "max_keys":
        return np.where(rng.random(n) < 0.4, np.uint32(0xFFFFFFFF), rng.integers(0, 2**32, n, dtype=np.uint32)).astype(np.uint32)
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["sorted", "reversed", "constant", "two_values", "sawtooth", "zipf16",
                                  "all_nan_and_zeros", "lognormal", "max_keys"])
def test_inputs_that_strain_the_splitters(abi, kind):
    rng = np.random.default_rng(74)
    for n in (33333, 262144 + 11):
        a = adversarial(kind, n, rng)
        print(f"bucket kind={kind} n={n}", flush=True)
        check(abi, a)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.int32, np.float32, np.int64, np.float64, np.complex64],
                         ids=lambda d: np.dtype(d).name)
def test_bins_too_long_for_the_registers(abi, dtype):
    """bucket_cap far below the bins' lengths: every bin goes through the workgroup's loop
    over global memory (bucket_sort_long); also few bins for a long row."""
    rng = np.random.default_rng(75)
    for n, bins, cap in ((40001, 4, 256), (100003, 2, 1024), (70001, 256, 64), (300007, 7, 0)):
        a = random_array(dtype, n, rng)
        print(f"bucket long bins dtype={np.dtype(dtype).name} n={n} bins={bins} cap={cap}", flush=True)
        check(abi, a, options=Options(bucket_path=1, bucket_bins=bins, bucket_cap=cap))
    pay = rng.integers(-2**62, 2**62, 40001, dtype=np.int64)
    a = random_array(dtype, 40001, rng)
    got = abi.local_sort(a, a.size, argsort=True, indices_in=pay, inplace=True,
                         options=Options(bucket_path=1, bucket_bins=3, bucket_cap=128))
    assert np.array_equal(got, pay[np.argsort(a, kind="stable")])


@pytest.mark.parametrize("dtype", [np.int16, np.int32, np.float32, np.int64, np.float64, np.complex64],
                         ids=lambda d: np.dtype(d).name)
def test_rows_of_several_million_elements_when_asked_for(abi, dtype):
    """Rows beyond what 256 bins of register size hold do not take this path by themselves;
    asked for, every bin is a few tiles long and is sorted tile by tile through global memory,
    and the scatter walks its largest tiles, several per chunk."""
    rng = np.random.default_rng(76)
    o = Options(bucket_path=1)
    for n in ((1 << 21) + 5, (1 << 22) + 4099):
        for narrow in (False, True):
            a = random_array(dtype, n, rng, narrow=narrow)
            print(f"bucket dtype={np.dtype(dtype).name} n={n} narrow={narrow} "
                  f"plan={abi.describe_plan(dtype, n, n, True, options=o)}", flush=True)
            assert "strategy=bucket" in abi.describe_plan(dtype, n, n, True, options=o)
            check(abi, a, options=o)
    pay = rng.integers(-2**62, 2**62, n, dtype=np.int64)
    got = abi.local_sort(a, n, argsort=True, indices_in=pay, inplace=True, options=o)
    assert np.array_equal(got, pay[np.argsort(a, kind="stable")])


@pytest.mark.parametrize("dtype", [np.int32, np.float64], ids=lambda d: np.dtype(d).name)
def test_uneven_bins_from_a_thin_sample(abi, dtype):
    """One sample key per bin: bin lengths spread like an exponential distribution, so that at
    a million elements a few bins outgrow the registers and take the loop through global
    memory, next to bins of a handful of elements."""
    rng = np.random.default_rng(78)
    for n in (1 << 20, 700001):
        a = random_array(dtype, n, rng)
        check(abi, a, options=Options(bucket_oversample=1))
        check(abi, a, options=Options(bucket_oversample=3, bucket_cap=2048))


@pytest.mark.parametrize("dtype", [np.int64, np.uint64, np.float64], ids=lambda d: np.dtype(d).name)
def test_sample_keys_that_agree_in_their_upper_bits(abi, dtype):
    """The sample of 8-byte keys is sorted by the 40 most significant bits that vary, and by all
    of them only if two sample keys agree in those and differ below: clusters far apart with
    small differences inside (every sample key has a neighbour like that), clusters next to
    unique keys, and keys that vary in exactly 40 and 41 bits."""
    rng = np.random.default_rng(79)
    n = 200001
    noise = rng.integers(0, 1 << 20, n)
    inputs = {}
    if np.dtype(dtype).kind == "f":
        inputs["two clusters"] = np.where(rng.integers(0, 2, n) == 0, 1.0, 1e300) * (1.0 + noise * 2.0**-52)
        inputs["clusters and unique"] = np.where(rng.integers(0, 4, n) == 0, 1.0 + noise * 2.0**-52, rng.standard_normal(n))
    else:
        far = np.array([0, 1 << 62, (1 << 62) + (1 << 45)], dtype=np.uint64)
        inputs["three clusters"] = (far[rng.integers(0, 3, n)] + noise.astype(np.uint64)).astype(dtype)
        inputs["40 bits"] = rng.integers(0, 1 << 40, n).astype(dtype)
        inputs["41 bits"] = rng.integers(0, 1 << 41, n).astype(dtype)
        inputs["clusters and unique"] = np.where(rng.integers(0, 4, n) == 0, noise, rng.integers(0, 1 << 62, n)).astype(dtype)
    for name, a in inputs.items():
        a = a.astype(dtype)
        print(f"bucket upper bits dtype={np.dtype(dtype).name} case={name}", flush=True)
        assert "strategy=bucket" in abi.describe_plan(dtype, n, n, True)
        check(abi, a)


def test_path_can_be_switched_off_per_call(abi):
    rng = np.random.default_rng(77)
    a = random_array(np.float32, 50001, rng)
    check(abi, a, options=Options(bucket_path=0))


def test_ballot_rank_gives_the_same_sort():
    """A fresh process with MISORT_RANK_BALLOT=1: the same path ranked by ballots only."""
    code = r"""
import numpy as np, sys
sys.path.insert(0, %r)
from tests.util import Abi, random_array
from cunumeric_amd._lib import Options
abi = Abi()
assert abi.lib.misort_rank_mode() == 2
rng = np.random.default_rng(5)
for dtype, n in ((np.float32, 300001), (np.int64, 200003), (np.uint16, 70001), (np.complex64, 33333)):
    for narrow in (False, True):
        a = random_array(dtype, n, rng, narrow=narrow)
        assert "strategy=bucket" in abi.describe_plan(dtype, n, n, True)
        assert np.array_equal(abi.local_sort(a, n, argsort=True), np.argsort(a, kind="stable")), dtype
        assert abi.local_sort(a, n, argsort=False).tobytes() == np.sort(a, kind="stable").tobytes(), dtype
a = random_array(np.int32, 50001, rng)
o = Options(bucket_path=1, bucket_bins=3, bucket_cap=128)
assert np.array_equal(abi.local_sort(a, a.size, argsort=True, options=o), np.argsort(a, kind="stable"))
print("ballot ok")
""" % ROOT
    env = dict(os.environ, MISORT_RANK_BALLOT="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ballot ok" in r.stdout
