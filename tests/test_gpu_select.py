"""misort_select: order statistics of every row without moving the row.

Checked against numpy.sort of the same rows: the element at kth, the one at kth + 1 and the
last one, for six element types, rows with heavy ties, rows whose leading key bytes are
constant (so that the keys that still match are written out late or never), NaNs, signed
zeros and infinities.  Floating-point results are compared as values (a zero comes back as +0
and a NaN as the default NaN, which is what the entry point documents)."""
import numpy as np
import pytest

from oracle import misort_oracle as oracle
from tests.util import Abi, random_array

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    return Abi()


def select(abi, a, kth, want_next=True, want_max=True, want_kth=True):
    import torch

    a = np.ascontiguousarray(a)
    rows, n = (1, a.size) if a.ndim == 1 else a.shape
    code = abi.to_code(a.dtype)
    need = abi.lib.misort_select_scratch_bytes(code, a.size, n, kth)
    assert need > 0
    d_in = torch.from_numpy(a.reshape(-1).view(np.uint8).copy()).to(abi.dev)
    scratch = torch.empty(need, dtype=torch.uint8, device=abi.dev)
    outs = [torch.zeros(rows * a.dtype.itemsize, dtype=torch.uint8, device=abi.dev) if w else None
            for w in (want_kth, want_next, want_max)]
    rc = abi.lib.misort_select(code, d_in.data_ptr(), a.size, n, kth, *[o.data_ptr() if o is not None else None
                                                                        for o in outs],
                               scratch.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, abi.lib.misort_last_error()
    torch.cuda.synchronize()
    assert bytes(d_in.cpu().numpy()) == a.tobytes()  # the rows are read, not written
    return [o.cpu().numpy().view(a.dtype) if o is not None else None for o in outs]


def same_values(got, ref):
    return np.array_equal(got, ref, equal_nan=True)


DTYPES = [np.int32, np.uint32, np.float32, np.int64, np.uint64, np.float64]


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: np.dtype(d).name)
def test_against_a_sort(abi, dtype):
    rng = np.random.default_rng(61)
    for n, narrow in ((100003, False), (100003, True), (1 << 20, False)):
        a = random_array(dtype, n, rng, narrow=narrow)
        s = np.sort(a)
        for kth in (0, 1, n // 3, n // 2, n - 2):
            print(f"select dtype={np.dtype(dtype).name} n={n} narrow={narrow} kth={kth}", flush=True)
            k, nxt, top = select(abi, a, kth)
            assert same_values(k, s[kth:kth + 1])
            assert same_values(nxt, s[kth + 1:kth + 2])
            assert same_values(top, s[-1:])
        k, nxt, top = select(abi, a, n - 1, want_next=False)
        assert nxt is None and same_values(k, s[-1:]) and same_values(top, s[-1:])
        k, nxt, top = select(abi, a, n // 7, want_next=False, want_max=False)
        assert same_values(k, s[n // 7:n // 7 + 1])


@pytest.mark.parametrize("dtype", [np.uint32, np.int64, np.float64], ids=lambda d: np.dtype(d).name)
def test_rows_that_narrow_down_at_different_passes(abi, dtype):
    rng = np.random.default_rng(62)
    n = 200003
    bits = np.dtype(dtype).itemsize * 8
    rows = [
        rng.integers(0, 2**(bits - 1), n, dtype=np.uint64),
        rng.integers(0, 2**16, n, dtype=np.uint64) + (1 << (bits - 3)),
        rng.integers(0, 2**24, n, dtype=np.uint64) << np.uint64(8),
        rng.integers(0, 3, n, dtype=np.uint64) * 77,
        np.where(rng.random(n) < 0.6, 12345, rng.integers(0, 2**(bits - 1), n, dtype=np.uint64)),
        np.full(n, 5, dtype=np.uint64),
    ]
    a = np.stack(rows).astype(np.uint64)
    a = a.astype(dtype) if np.dtype(dtype).kind != "f" else (a.astype(np.float64) - 2.0**40)
    s = np.sort(a, axis=1)
    for kth in (0, 7, n // 5, n // 2, n - 2):
        print(f"select rows dtype={np.dtype(dtype).name} kth={kth}", flush=True)
        k, nxt, top = select(abi, a, kth)
        assert same_values(k, s[:, kth]) and same_values(nxt, s[:, kth + 1]) and same_values(top, s[:, -1])


@pytest.mark.parametrize("dtype", [np.float32, np.int64], ids=lambda d: np.dtype(d).name)
def test_many_rows(abi, dtype):
    """Hundreds of rows just long enough for the selection: few chunks per row."""
    rng = np.random.default_rng(64)
    rows, n = 300, 66001
    a = random_array(dtype, rows * n, rng).reshape(rows, n)
    s = np.sort(a, axis=1)
    for kth in (0, n // 2, n - 2):
        k, nxt, top = select(abi, a, kth)
        assert same_values(k, s[:, kth]) and same_values(nxt, s[:, kth + 1]) and same_values(top, s[:, -1])


@pytest.mark.parametrize("dtype", [np.uint32, np.int32, np.float32, np.int64, np.float64],
                         ids=lambda d: np.dtype(d).name)
def test_next_element_lies_outside_the_keys_that_still_match(abi, dtype):
    """Keys spread so thinly that the kth key is the largest of those sharing its leading
    byte: the element after it is not among the keys the selection kept, and is found by
    reading the row once more."""
    rng = np.random.default_rng(65)
    n = 70001
    step = 60000 if np.dtype(dtype).itemsize == 4 else 1 << 46
    vals = (np.arange(n, dtype=np.int64) - (n // 2 if np.dtype(dtype).kind != "u" else 0)) * step
    if dtype == np.int32:
        vals //= 2
    a = np.stack([rng.permutation(vals).astype(dtype) for _ in range(3)])
    s = np.sort(a, axis=1)
    key = oracle.to_key(s[0])[-1]  # the sort keys of row 0, ascending
    shift = key.dtype.itemsize * 8 - 8
    last_of_bucket = np.nonzero((key[:-1] >> shift) != (key[1:] >> shift))[0]
    assert last_of_bucket.size >= 4
    for kth in [int(k) for k in last_of_bucket[:: max(1, last_of_bucket.size // 6)]] + [n - 2]:
        k, nxt, top = select(abi, a, kth)
        assert same_values(k, s[:, kth]) and same_values(nxt, s[:, kth + 1]) and same_values(top, s[:, -1]), kth


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.uint64], ids=lambda d: np.dtype(d).name)
def test_next_element_held_by_one_chunk_of_a_row_without_candidates(abi, dtype):
    """Rows of one repeated value plus a few larger ones: the keys that still match never
    become few enough to be written out, so the element after kth comes from the read of the
    row itself, and here the smallest larger value sits in the last chunk only while the
    first chunk holds a larger one.  Every workgroup of the row has to look at its chunk,
    whatever the others have already reported."""
    n = 600007
    for rep in range(3):
        a = np.full((2, n), 5, dtype=dtype)
        a[0, 3] = 900
        a[0, n - 2 - rep] = 7      # the answer, in the last chunk
        a[1, n - 5] = 901
        a[1, 11 + rep] = 8         # the answer, in the first chunk
        a[1, n // 2] = 4
        s = np.sort(a, axis=1)
        for kth in (n - 3, n - 4, 0):
            k, nxt, top = select(abi, a, kth)
            assert same_values(k, s[:, kth]) and same_values(nxt, s[:, kth + 1]) and same_values(top, s[:, -1]), kth


def test_nan_rows_and_signed_zeros(abi):
    rng = np.random.default_rng(63)
    n = 70001
    a = rng.standard_normal((4, n)).astype(np.float32)
    a[1, 17] = np.nan
    a[3, :] = np.where(rng.random(n) < 0.5, -0.0, 0.0)
    a[2, ::3] = -np.inf
    s = np.sort(a, axis=1)
    k, nxt, top = select(abi, a, n // 2)
    assert same_values(k, s[:, n // 2]) and same_values(nxt, s[:, n // 2 + 1])
    assert np.isnan(top[1]) and not np.isnan(top[[0, 2, 3]]).any()
    assert same_values(top, s[:, -1])
    # the position just before the NaN: the next element is the NaN
    k, nxt, _ = select(abi, a, n - 2)
    assert np.isnan(nxt[1]) and same_values(k, s[:, n - 2])


def test_what_is_not_served(abi):
    lib, code = abi.lib, abi.to_code
    n = 1 << 17
    assert lib.misort_select_scratch_bytes(code(np.dtype(np.int16)), n, n, 5) == 0
    assert lib.misort_select_scratch_bytes(code(np.dtype(np.complex64)), n, n, 5) == 0
    assert lib.misort_select_scratch_bytes(code(np.dtype(np.float32)), 4096, 64, 5) == 0  # short rows
    assert lib.misort_select_scratch_bytes(code(np.dtype(np.float32)), n, n, n) == 0  # kth outside the row
    assert lib.misort_select_scratch_bytes(code(np.dtype(np.float32)), n, n, -1) == 0
    import torch

    buf = torch.zeros(n * 4, dtype=torch.uint8, device=abi.dev)
    out = torch.zeros(16, dtype=torch.uint8, device=abi.dev)
    need = lib.misort_select_scratch_bytes(code(np.dtype(np.float32)), n, n, n - 1)
    scratch = torch.empty(need, dtype=torch.uint8, device=abi.dev)
    st = torch.cuda.current_stream().cuda_stream
    # nothing follows the last position
    assert lib.misort_select(code(np.dtype(np.float32)), buf.data_ptr(), n, n, n - 1, out.data_ptr(),
                             out.data_ptr(), None, scratch.data_ptr(), need, st) == 8
    assert lib.misort_select(code(np.dtype(np.int16)), buf.data_ptr(), n, n, 5, out.data_ptr(), None, None,
                             scratch.data_ptr(), need, st) == 8
    assert lib.misort_select(code(np.dtype(np.float32)), buf.data_ptr(), n, n, 5, out.data_ptr(), None, None,
                             scratch.data_ptr(), need - 256, st) == 4
    assert lib.misort_select(code(np.dtype(np.float32)), buf.data_ptr(), n, n, 5, None, None, None,
                             scratch.data_ptr(), need, st) == 2
    assert lib.misort_select(code(np.dtype(np.float32)), buf.data_ptr(), 0, n, 5, None, None, None, None, 0, st) == 0
    torch.cuda.synchronize()
