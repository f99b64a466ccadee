"""Randomly drawn cases on the radix and selection paths, each checked against NumPy:
partition / argpartition (the contract), misort_select (elements kth, kth + 1 and last of a
stable sort), sort (bit-exact) and stable argsort (exact), over element types, row counts,
row lengths off every alignment and key distributions that steer the kernels differently:
full range, few values, pools of repeated values (runs of equal keys in the later passes),
small ranges (dead leading bytes), sorted input, one value holding most of the row, small values
of both signs."""
import numpy as np
import pytest

import cunumeric_amd as num
from tests.test_gpu_partition_select import assert_partitioned
from tests.test_gpu_select import same_values, select
from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu

DTYPES = [np.int32, np.uint32, np.float32, np.int64, np.uint64, np.float64]


def draw(rng, dtype, rows, n, kind):
    total = rows * n
    if kind == 0:
        a = random_array(dtype, total, rng)
    elif kind == 1:
        a = random_array(dtype, total, rng, narrow=True)
    elif kind == 2:
        pool = random_array(dtype, max(2, total // int(rng.choice([16, 64, 256, 4096]))), rng, specials=False)
        a = pool[rng.integers(0, pool.size, total)]
    elif kind == 3:
        a = rng.integers(0, 1 << int(rng.choice([8, 12, 16, 20, 24])), total).astype(dtype)
    elif kind == 4:
        a = np.sort(random_array(dtype, total, rng, specials=False))
        if rng.integers(0, 2):
            a = a[::-1].copy()
    elif kind == 5:
        a = random_array(dtype, total, rng, specials=False)
        a[rng.random(total) < 0.7] = a[0]
    else:
        r = int(rng.choice([1, 100, 40000, 1 << 20]))
        off = int(rng.choice([0, 0, -r, 1 << 28, -(1 << 29)]))
        a = rng.integers(-r, r, total, endpoint=True) + off
        a = np.abs(a).astype(dtype) if np.dtype(dtype).kind == "u" else a.astype(dtype)
    return np.ascontiguousarray(a).reshape(rows, n)


@pytest.mark.parametrize("seed", range(6))
def test_random_cases(seed):
    abi = Abi()
    rng = np.random.default_rng(1000 + seed)
    for it in range(12):
        dtype = DTYPES[rng.integers(0, len(DTYPES))]
        rows = int(rng.choice([1, 1, 2, 3, 7, 20]))
        n = int(rng.choice([65536, 65537, 70001, 100003, 131072, 200001, 262144 + 5, 500009]))
        rows = min(rows, max(1, 3_000_000 // n))
        kind = int(rng.integers(0, 7))
        a = draw(rng, dtype, rows, n, kind)
        kth = int(rng.choice([0, 1, n // 2, n - 2, n - 1, int(rng.integers(0, n))]))
        tag = f"seed={seed} it={it} dtype={np.dtype(dtype).name} rows={rows} n={n} kind={kind} kth={kth}"
        print(tag, flush=True)
        s = np.sort(a, axis=1, kind="stable")
        assert_partitioned(a, np.asarray(num.partition(a, kth, axis=1)), kth)
        idx = np.asarray(num.argpartition(a, kth, axis=1))
        assert np.array_equal(np.sort(idx, axis=1), np.broadcast_to(np.arange(n), a.shape)), tag
        assert_partitioned(a, np.take_along_axis(a, idx, axis=1), kth)
        if kth + 1 < n:
            k, nxt, top = select(abi, a, kth)
            assert same_values(k, s[:, kth]) and same_values(nxt, s[:, kth + 1]), tag
            assert same_values(top, s[:, -1]), tag
        got = np.asarray(num.sort(a, axis=1))
        assert bits_equal(got, s) or np.array_equal(got, s, equal_nan=True), tag
        assert np.array_equal(np.asarray(num.argsort(a, axis=1, kind="stable")),
                              np.argsort(a, axis=1, kind="stable")), tag
