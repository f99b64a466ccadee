"""partition / argpartition by selection (long rows of 4-byte and wider elements).

The property checked is NumPy's contract (and what the reference's test_partition.py
asserts, tests/integration/test_partition.py:23-67): the element at kth is the one a full
sort puts there, nothing larger stands before it, nothing smaller after it; for
argpartition the same of the gathered elements, and the positions are a permutation."""
import numpy as np
import pytest

import cunumeric_amd as num
from oracle import misort_oracle as oracle
from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    return Abi()


def assert_partitioned(a, out, kth, axis=-1):
    a = np.moveaxis(np.asarray(a), axis, -1)
    out = np.moveaxis(np.asarray(out), axis, -1)
    assert out.shape == a.shape and out.dtype == a.dtype
    srt = np.sort(a, axis=-1, kind="stable")
    # same multiset per row
    assert bits_equal(np.sort(out, axis=-1, kind="stable"), srt) or np.array_equal(
        np.sort(out, axis=-1, kind="stable"), srt, equal_nan=True)
    ka = oracle.to_key(np.ascontiguousarray(out).reshape(-1, out.shape[-1]))
    ks = oracle.to_key(np.ascontiguousarray(srt).reshape(-1, srt.shape[-1]))
    for w_out, w_srt in [(ka, ks)]:
        hi_o, hi_s = w_out[-1], w_srt[-1]
        if len(w_out) == 1:
            piv = hi_s[:, kth][:, None]
            assert np.all(hi_o[:, kth] == hi_s[:, kth])
            assert np.all(hi_o[:, :kth] <= piv) and np.all(hi_o[:, kth + 1:] >= piv)
        else:
            lo_o, lo_s = w_out[0], w_srt[0]
            ph, pl = hi_s[:, kth][:, None], lo_s[:, kth][:, None]
            assert np.all((hi_o[:, kth] == hi_s[:, kth]) & (lo_o[:, kth] == lo_s[:, kth]))
            le = (hi_o < ph) | ((hi_o == ph) & (lo_o <= pl))
            ge = (hi_o > ph) | ((hi_o == ph) & (lo_o >= pl))
            assert np.all(le[:, :kth]) and np.all(ge[:, kth + 1:])


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32, np.int64, np.uint64, np.float64,
                                   np.complex64, np.complex128], ids=lambda d: np.dtype(d).name)
def test_partition_and_argpartition_long_rows(dtype):
    rng = np.random.default_rng(51)
    for n, narrow in ((20000, False), (100003, False), (100003, True), (1 << 20, False)):
        a = random_array(dtype, n, rng, narrow=narrow)
        for kth in (0, 1, n // 3, n - 1, -1):
            k = kth % n
            print(f"partition dtype={np.dtype(dtype).name} n={n} narrow={narrow} kth={kth}", flush=True)
            assert_partitioned(a, num.partition(a, kth), k)
            idx = np.asarray(num.argpartition(a, kth))
            assert idx.dtype == np.int64 and np.array_equal(np.sort(idx), np.arange(n))
            assert_partitioned(a, a[idx], k)
        b = num.array(a)
        b.partition(n // 2)
        assert_partitioned(a, b, n // 2)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128],
                         ids=lambda d: np.dtype(d).name)
def test_values_keep_their_bit_patterns(dtype):
    """The split moves the values as they came in: NaN payloads and signed zeros survive."""
    rng = np.random.default_rng(55)
    n = 120001
    a = random_array(dtype, n, rng)
    size = a.dtype.itemsize

    def bit_patterns(x):
        raw = np.ascontiguousarray(x).tobytes()
        return sorted(raw[i:i + size] for i in range(0, len(raw), size))

    want = bit_patterns(a)
    for kth in (0, n // 2, n - 1):
        out = np.asarray(num.partition(a, kth))
        assert_partitioned(a, out, kth)
        assert bit_patterns(out) == want
    b = num.array(a)
    b.partition(n // 3)
    assert bit_patterns(np.asarray(b)) == want


@pytest.mark.parametrize("dtype", [np.float32, np.int64], ids=lambda d: np.dtype(d).name)
def test_many_rows(dtype):
    """Hundreds of rows just long enough for the selection: few chunks per row."""
    rng = np.random.default_rng(56)
    rows, n = 300, 66001
    a = random_array(dtype, rows * n, rng).reshape(rows, n)
    for kth in (0, n // 2, n - 1):
        assert_partitioned(a, num.partition(a, kth, axis=1), kth)
        idx = np.asarray(num.argpartition(a, kth, axis=1))
        assert np.array_equal(np.sort(idx, axis=1), np.broadcast_to(np.arange(n), a.shape))
        assert_partitioned(a, np.take_along_axis(a, idx, axis=1), kth)


def test_rows_axes_and_fallbacks():
    rng = np.random.default_rng(52)
    a = rng.standard_normal((3, 70001)).astype(np.float32)
    assert_partitioned(a, num.partition(a, 500, axis=-1), 500)
    idx = np.asarray(num.argpartition(a, 500, axis=1))
    assert_partitioned(a, np.take_along_axis(a, idx, axis=1), 500)
    c = rng.integers(-1000, 1000, (40000, 3)).astype(np.int64)
    assert_partitioned(c, num.partition(c, 123, axis=0), 123, axis=0)
    idx = np.asarray(num.argpartition(c, 123, axis=0))
    assert_partitioned(c, np.take_along_axis(c, idx, axis=0), 123, axis=0)
    flat = num.partition(c, 77, axis=None)
    assert_partitioned(c.reshape(-1), flat, 77)
    # a sequence of positions and an out-of-range position sort completely, as the reference does
    d = rng.standard_normal(50000)
    assert np.array_equal(np.asarray(num.partition(d, (5, 100))), np.sort(d))
    assert np.array_equal(np.asarray(num.partition(d, 10**9)), np.sort(d))


@pytest.mark.parametrize("dtype", [np.uint32, np.int64, np.float64], ids=lambda d: np.dtype(d).name)
def test_rows_that_narrow_down_at_different_passes(dtype):
    """The selection writes the keys that still match side by side once they are few and reads
    only those afterwards; when that happens depends on the row: at once (all bytes vary), after
    some passes (leading bytes equal), never (few distinct values), or only for some ranks
    (one heavy value beside spread-out ones)."""
    rng = np.random.default_rng(54)
    n = 300007
    bits = np.dtype(dtype).itemsize * 8
    rows = [
        rng.integers(0, 2**(bits - 1), n, dtype=np.uint64),            # every byte varies
        rng.integers(0, 2**16, n, dtype=np.uint64) + (1 << (bits - 3)),  # only the low two bytes
        rng.integers(0, 2**24, n, dtype=np.uint64) << np.uint64(8),     # the lowest byte is constant
        rng.integers(0, 3, n, dtype=np.uint64) * 77,                     # three values
        np.where(rng.random(n) < 0.6, 12345, rng.integers(0, 2**(bits - 1), n, dtype=np.uint64)),
    ]
    a = np.stack(rows).astype(np.uint64)
    a = a.astype(dtype) if np.dtype(dtype).kind != "f" else (a.astype(np.float64) - 2.0**40)
    for kth in (0, 7, n // 5, n // 2, n - 2):
        print(f"narrowing dtype={np.dtype(dtype).name} kth={kth}", flush=True)
        assert_partitioned(a, num.partition(a, kth, axis=1), kth)
        idx = np.asarray(num.argpartition(a, kth, axis=1))
        assert np.array_equal(np.sort(idx, axis=1), np.broadcast_to(np.arange(n), a.shape))
        assert_partitioned(a, np.take_along_axis(a, idx, axis=1), kth)


def test_c_abi_plan_and_offset(abi):
    """the C entry point directly: positions carry index_offset; 2-byte values still count"""
    import torch

    rng = np.random.default_rng(53)
    n = 150001
    a = rng.integers(-2**31, 2**31, n, dtype=np.int32)
    dev = abi.dev
    d_in = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_idx = torch.empty(n * 8, dtype=torch.uint8, device=dev)
    code = abi.to_code(a.dtype)
    kth, off = 4242, 1000
    need = abi.lib.misort_partition_scratch_bytes(code, n, n, 1, kth)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    rc = abi.lib.misort_partition(code, d_in.data_ptr(), None, d_idx.data_ptr(), n, n, kth, off,
                                  scratch.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    idx = d_idx.cpu().numpy().view(np.int64) - off
    assert np.array_equal(np.sort(idx), np.arange(n))
    assert_partitioned(a, a[idx], kth)
    # in place, values
    need = abi.lib.misort_partition_scratch_bytes(code, n, n, 0, kth)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    rc = abi.lib.misort_partition(code, d_in.data_ptr(), d_in.data_ptr(), None, n, n, kth, 0,
                                  scratch.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert_partitioned(a, d_in.cpu().numpy().view(np.int32), kth)
