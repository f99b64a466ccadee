"""searchsorted on the GPU against numpy.searchsorted.

The case tables restate the reference's integration test
(tests/integration/test_searchsorted.py:29-53, 197-244: standard dtypes and volumes,
mixed-dtype pairs, both sides, a sorter from argsort, v of 0 to 4 dimensions, empty inputs,
shape errors); on top of that: ties, special floating-point values, and sizes that need the
two-level search."""
import numpy as np
import pytest

import cunumeric_amd as num
from tests.util import random_array

pytestmark = pytest.mark.gpu

SIDES = ["left", "right"]

STANDARD_CASES = [
    (156, np.uint8), (123, np.uint16), (241, np.uint32), (1, np.uint64), (21, np.int8),
    (5, np.int16), (34, np.int32), (11, np.int64), (31, np.float32), (11, np.float64),
    (422, np.double), (220, np.double), (244, np.complex64), (24, np.complex128),
    (220, np.complex128), (0, np.uint32),
]

DTYPE_CASES = [
    (3, np.uint64, np.float32), (51, np.uint32, np.complex64), (23, np.uint32, np.float64),
    (51, np.complex64, np.float64), (21, np.complex64, np.int32), (22, np.complex128, np.float32),
]


def generate_random(volume, datatype, rng):
    dt = np.dtype(datatype)
    if dt.kind in "iu":
        ii = np.iinfo(dt)
        return rng.integers(ii.min, ii.max, size=volume, dtype=dt)
    if dt.kind == "f":
        return rng.random(volume).astype(dt)
    return (rng.random(volume) + rng.random(volume) * 1j).astype(dt)


def check_api(a, rng, dtype2=None, v=None, side="left"):
    a_argsorted = np.argsort(a, kind="stable")
    if v is None:
        v = generate_random(10, dtype2 if dtype2 is not None else a.dtype, rng)
    a_num, v_num, s_num = num.array(a), num.array(v), num.array(a_argsorted)

    res_np = a.searchsorted(v, side=side, sorter=a_argsorted)
    res_num = a_num.searchsorted(v_num, side=side, sorter=s_num)
    assert np.array_equal(res_np, np.asarray(res_num))
    assert np.asarray(res_num).dtype == np.int64 and np.asarray(res_num).shape == np.shape(v)

    res_num = num.searchsorted(a_num, v_num, side=side, sorter=s_num)
    assert np.array_equal(np.searchsorted(a, v, side=side, sorter=a_argsorted), np.asarray(res_num))


@pytest.mark.parametrize("side", SIDES)
def test_empty_v(side):
    rng = np.random.default_rng(1)
    check_api(np.arange(25), rng, None, np.arange(0), side)
    check_api(np.array([]), rng, side=side)
    check_api(np.arange(0), rng, None, np.arange(0), side=side)


@pytest.mark.parametrize("volume, dtype1, dtype2", DTYPE_CASES, ids=str)
@pytest.mark.parametrize("side", SIDES)
def test_dtype_conversions(volume, dtype1, dtype2, side):
    rng = np.random.default_rng(2)
    check_api(generate_random(volume, dtype1, rng), rng, dtype2, side=side)


@pytest.mark.parametrize("volume, dtype", STANDARD_CASES, ids=str)
@pytest.mark.parametrize("side", SIDES)
def test_standard_cases(volume, dtype, side):
    rng = np.random.default_rng(3)
    check_api(generate_random(volume, dtype, rng), rng, side=side)


@pytest.mark.parametrize("ndim", range(0, 5))
@pytest.mark.parametrize("side", SIDES)
def test_ndim(ndim, side):
    rng = np.random.default_rng(4)
    a = rng.integers(-100, 100, size=100)
    v = rng.integers(-100, 100, size=2**ndim).reshape(tuple(2 for _ in range(ndim)))
    check_api(a, rng, None, v, side)


def test_scalar_and_errors():
    a = np.sort(np.random.default_rng(5).integers(-50, 50, 200))
    for side in SIDES:
        got = num.searchsorted(a, 7, side=side)
        assert isinstance(got, int) and got == int(np.searchsorted(a, 7, side=side))
    with pytest.raises(ValueError):
        num.searchsorted(np.zeros((5, 5, 5)), 5)
    with pytest.raises(ValueError):
        num.searchsorted(a, [1, 2], sorter=np.arange(10))
    with pytest.raises(ValueError):
        num.searchsorted(a, [1, 2], sorter=np.zeros((5, 5, 5), dtype=np.int64))
    with pytest.raises(ValueError):
        num.searchsorted(a, [1, 2], sorter=np.zeros(a.shape, dtype=np.float64))
    with pytest.raises(ValueError):
        num.searchsorted(a, 10, "hi")


@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.int32, np.float16, np.float32, np.float64,
                                   np.int64, np.complex64, np.complex128], ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("side", SIDES)
def test_ties_specials_and_long_arrays(dtype, side):
    """Sorted by this library (so NaN / -0 / complex tiers sit where NumPy puts them);
    queries drawn from the array itself (ties) and from fresh values incl. specials."""
    rng = np.random.default_rng(6)
    for n in (1, 2, 1000, 1024, 1025, 70001, 1 << 21):
        a = np.asarray(num.sort(random_array(dtype, n, rng, narrow=(n == 1000))))
        v = np.concatenate([a[rng.integers(0, n, 300)], random_array(dtype, 300, rng)])
        print(f"searchsorted dtype={np.dtype(dtype).name} n={n} side={side}", flush=True)
        got = np.asarray(num.searchsorted(a, v, side=side))
        assert np.array_equal(got, np.searchsorted(a, v, side=side)), (dtype, n, side)


# ---- many queries into a large array: the library sorts the queries first (workspace entry
# point) and stores every answer where its query came from ----

def _reference_positions(a_sorted, v, side):
    """numpy.searchsorted; for float16 / complex data with NaNs NumPy's own ordering of the
    array and of the queries is the same one the library uses (NaN last, tiers for complex)."""
    return np.searchsorted(a_sorted, v, side=side)


@pytest.mark.parametrize("side", SIDES)
@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.int32, np.float32, np.int64, np.float64,
                                   np.complex64, np.complex128], ids=lambda d: np.dtype(d).name)
def test_many_queries_large_array(dtype, side):
    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    dt = np.dtype(dtype)
    rng = np.random.default_rng(71)
    n = (64 << 20) // dt.itemsize + 1001          # just past the size from which queries are sorted
    m = (1 << 20) + 77
    a = np.sort(random_array(dtype, n, rng, specials=True), kind="stable")
    v = random_array(dtype, m, rng, specials=True)
    v[: m // 8] = a[rng.integers(0, n, m // 8)]   # exact hits, so the two sides differ
    assert _lib.load().misort_searchsorted_scratch_bytes(to_core_dtype(dt), n, m) > 0
    print(f"searchsorted sorted queries dtype={dt.name} side={side}", flush=True)
    got = np.asarray(num.searchsorted(num.array(a), num.array(v), side=side))
    assert got.dtype == np.int64 and got.shape == v.shape
    assert np.array_equal(got, _reference_positions(a, v, side))


def test_workspace_entry_point_matches_the_plain_one():
    """The same call with and without a workspace through the C ABI, 2-D queries."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    rng = np.random.default_rng(72)
    n, m = (1 << 24) + 5, (1 << 20) + 3
    a = np.sort(rng.standard_normal(n).astype(np.float32))
    v = rng.standard_normal(m).astype(np.float32)
    v[::7] = np.nan
    v[1::7] = -0.0
    dev = torch.device("cuda", 0)
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_v = torch.from_numpy(v.view(np.uint8)).to(dev)
    code = to_core_dtype(np.dtype(np.float32))
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for with_ws in (False, True):
        for left in (1, 0):
            d_o = torch.full((m,), -1, dtype=torch.int64, device=dev)
            need = lib.misort_searchsorted_scratch_bytes(code, n, m) if with_ws else 0
            assert (need > 0) == with_ws
            d_s = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
            _lib.check(lib.misort_searchsorted_ws(code, d_a.data_ptr(), n, d_v.data_ptr(), m, left,
                                                  d_o.data_ptr(), d_s.data_ptr() if with_ws else None, need, stream))
            torch.cuda.synchronize()
            outs.append(d_o.cpu().numpy())
    assert np.array_equal(outs[0], outs[2]) and np.array_equal(outs[1], outs[3])
    assert np.array_equal(outs[0], np.searchsorted(a, v, side="left"))
    assert np.array_equal(outs[1], np.searchsorted(a, v, side="right"))
    # too small a workspace is refused before anything runs
    d_o = torch.empty(m, dtype=torch.int64, device=dev)
    d_s = torch.empty(4096, dtype=torch.uint8, device=dev)
    rc = lib.misort_searchsorted_ws(code, d_a.data_ptr(), n, d_v.data_ptr(), m, 1, d_o.data_ptr(),
                                    d_s.data_ptr(), 4096, stream)
    assert rc == 4   # MISORT_ERR_SCRATCH


@pytest.mark.parametrize("side", SIDES)
def test_many_queries_degenerate_shapes(side):
    """Query sets whose sorted form gives a workgroup an empty or a one-sided stretch of the
    array: all queries equal (inside a long run of ties), all below the first element, all
    above the last, all NaN, already sorted, reversed."""
    rng = np.random.default_rng(73)
    n, m = (1 << 24) + 5, (1 << 20) + 3
    a = np.sort(np.round(rng.standard_normal(n) * 50).astype(np.float32))   # long runs of ties
    a_num = num.array(a)
    base = rng.standard_normal(m).astype(np.float32) * 50
    cases = {
        "all equal": np.full(m, 7.0, dtype=np.float32),
        "all below": np.full(m, -1e9, dtype=np.float32),
        "all above": np.full(m, 1e9, dtype=np.float32),
        "all nan": np.full(m, np.nan, dtype=np.float32),
        "sorted": np.sort(base),
        "reversed": np.sort(base)[::-1].copy(),
        "two far values": np.where(rng.integers(0, 2, m) == 0, np.float32(-1e9), np.float32(1e9)).astype(np.float32),
    }
    for name, v in cases.items():
        print(f"searchsorted degenerate case={name} side={side}", flush=True)
        got = np.asarray(num.searchsorted(a_num, num.array(v), side=side))
        assert np.array_equal(got, np.searchsorted(a, v, side=side)), name
