"""GPU tests of the Python surface: cunumeric_amd.sort / argsort / msort / sort_complex /
partition / argpartition and the ndarray methods.

These restate the reference's own sort tests (tests/integration/test_sort.py,
test_argsort.py, test_msort.py, test_sort_complex.py, test_partition.py of cuNumeric):
same shape matrix, same axis sweep, same kinds, same exceptions; NumPy is the oracle, as it
is there.  Where the reference leaves a case untested (NaN, signed zeros, the other 12
dtypes, in-place sort on a non-last axis) NumPy alone pins the expected result.
"""
import numpy as np
import pytest

import cunumeric_amd as num
from tests.util import ALL_DTYPES, bits_equal, random_array

pytestmark = pytest.mark.gpu

DIM = 5
SIZES = [
    (0,), (1), (DIM), (0, 1), (1, 0), (1, 1), (1, DIM), (DIM, 1), (DIM, DIM), (1, 0, 0),
    (1, 1, 0), (1, 0, 1), (1, 1, 1), (DIM, 1, 1), (1, DIM, 1), (1, 1, DIM), (DIM, DIM, DIM),
]
SORT_TYPES = ["quicksort", "mergesort", "heapsort", "stable"]
STABLE_SORT_TYPES = ["stable", "mergesort"]
UNSTABLE_SORT_TYPES = ["heapsort", "quicksort"]


def rint(rng, size):
    return rng.integers(-100, 100, size)


def rcomplex(rng, size):
    return rng.integers(-100, 100, size) + rng.integers(-100, 100, size) * 1.0j


# ---- test_sort.py ---------------------------------------------------------------------
class TestSort:
    @pytest.mark.parametrize("arr", ([], [[]], [[], []]))
    def test_arr_empty(self, arr):
        assert np.array_equal(num.sort(arr), np.sort(arr))

    def test_axis_out_bound(self):
        with pytest.raises(ValueError):
            num.sort([-1, 0, 1, 2, 10], axis=2)

    def test_sorttype_invalid_is_accepted(self):
        # the reference accepts any kind string (xfail test_sorttype_invalid): so do we
        a = np.random.default_rng(0).integers(-3, 3, (3, 3, 2))
        assert np.array_equal(num.sort(a, kind="negative"), np.sort(a))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_basic_axis(self, size):
        a = rint(np.random.default_rng(1), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(num.sort(a_num, axis=axis), np.sort(a, axis=axis))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", SORT_TYPES)
    def test_basic_axis_sort_type(self, size, sort_type):
        a = rint(np.random.default_rng(2), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(num.sort(a_num, axis=axis, kind=sort_type),
                                  np.sort(a, axis=axis, kind=sort_type))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", SORT_TYPES)
    def test_arr_basic_axis_inplace(self, size, sort_type):
        # skipped in the reference for a known bug; NumPy's in-place semantics are the rule
        a = rint(np.random.default_rng(3), size)
        for axis in range(-a.ndim + 1, a.ndim):
            a_num = num.array(a)
            a_np = a.copy()
            a_num.sort(axis=axis, kind=sort_type)
            a_np.sort(axis=axis, kind=sort_type)
            assert np.array_equal(a_num, a_np)

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", SORT_TYPES)
    def test_basic_complex_axis_sort(self, size, sort_type):
        a = rcomplex(np.random.default_rng(4), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(num.sort(a_num, axis=axis, kind=sort_type),
                                  np.sort(a, axis=axis, kind=sort_type))

    def test_axis_none_flattens(self):
        a = rint(np.random.default_rng(5), (4, 3, 5))
        res = num.sort(a, axis=None)
        assert res.shape == (60,)
        assert np.array_equal(res, np.sort(a, axis=None))

    def test_order_not_supported(self):
        with pytest.raises(NotImplementedError):
            num.sort([3, 1, 2], order="x")

    def test_unsupported_dtype(self):
        with pytest.raises(TypeError):
            num.sort(np.array(["b", "a"]))


# ---- test_argsort.py ------------------------------------------------------------------
class TestArgSort:
    @pytest.mark.parametrize("arr", ([], [[]], [[], []]))
    def test_arr_empty(self, arr):
        assert np.array_equal(num.argsort(arr), np.argsort(arr))

    def test_axis_out_bound(self):
        with pytest.raises(ValueError):
            num.argsort([-1, 0, 1, 2, 10], axis=2)

    def test_structured_array_order(self):
        a = np.array([(1, 2), (0, 1)], dtype=[("x", "<i4"), ("y", "<i4")])
        with pytest.raises((NotImplementedError, TypeError)):
            num.argsort(a, order=("x", "y"))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_basic_axis(self, size):
        # default kind with ties: the reference expects NumPy's answer; ours is always the
        # stable one, which is what NumPy's default returns for these sizes
        a = rint(np.random.default_rng(6), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            res = num.argsort(a_num, axis=axis)
            assert res.dtype == np.int64
            assert np.array_equal(res, np.argsort(a, axis=axis, kind="stable"))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", STABLE_SORT_TYPES)
    def test_basic_axis_sort_type(self, size, sort_type):
        a = rint(np.random.default_rng(7), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(num.argsort(a_num, axis=axis, kind=sort_type),
                                  np.argsort(a, axis=axis, kind=sort_type))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", UNSTABLE_SORT_TYPES)
    def test_basic_axis_sort_type_unstable(self, size, sort_type):
        # unique values, as in the reference (unstable kinds on ties are not comparable)
        rng = np.random.default_rng(8)
        a = np.arange(int(np.prod(size)))
        rng.shuffle(a)
        a = a.reshape(size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            res = np.asarray(num.argsort(a_num, axis=axis, kind=sort_type))
            assert np.array_equal(res, np.argsort(a, axis=axis, kind=sort_type))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", SORT_TYPES)
    def test_unstable_kinds_with_ties_are_permutations(self, size, sort_type):
        a = rint(np.random.default_rng(9), size)
        for axis in range(-a.ndim + 1, a.ndim):
            idx = np.asarray(num.argsort(a, axis=axis, kind=sort_type))
            assert np.array_equal(np.sort(idx, axis=axis),
                                  np.broadcast_to(
                                      np.arange(a.shape[axis]).reshape(
                                          [-1 if i == axis % a.ndim else 1 for i in range(a.ndim)]),
                                      a.shape)) if a.size else True
            assert np.array_equal(np.take_along_axis(a, idx, axis=axis), np.sort(a, axis=axis))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_arr_basic_axis(self, size):
        a = rint(np.random.default_rng(10), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(a_num.argsort(axis=axis), a.argsort(axis=axis, kind="stable"))

    @pytest.mark.parametrize("size", SIZES, ids=str)
    @pytest.mark.parametrize("sort_type", STABLE_SORT_TYPES)
    def test_basic_complex_axis_sort_type(self, size, sort_type):
        a = rcomplex(np.random.default_rng(11), size)
        a_num = num.array(a)
        for axis in range(-a.ndim + 1, a.ndim):
            assert np.array_equal(num.argsort(a_num, axis=axis, kind=sort_type),
                                  np.argsort(a, axis=axis, kind=sort_type))

    def test_axis_none(self):
        a = rint(np.random.default_rng(12), (3, 4, 5))
        res = num.argsort(a, axis=None, kind="stable")
        assert res.shape == (60,)
        assert np.array_equal(res, np.argsort(a, axis=None, kind="stable"))


# ---- test_msort.py / test_sort_complex.py ---------------------------------------------
class TestMsortSortComplex:
    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_msort(self, size):
        a = rint(np.random.default_rng(13), size)
        assert np.array_equal(num.msort(a), np.sort(a, axis=0))
        c = rcomplex(np.random.default_rng(14), size)
        assert np.array_equal(num.msort(c), np.sort(c, axis=0))

    @pytest.mark.parametrize("arr", ([], [[]], [[], []]))
    def test_sort_complex_empty(self, arr):
        assert np.array_equal(num.sort_complex(arr), np.sort_complex(arr))

    @pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32])
    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_sort_complex_promotion(self, size, dtype):
        a = np.random.default_rng(15).integers(-100, 100, size, dtype=dtype)
        res = num.sort_complex(num.array(a))
        ref = np.sort_complex(a)
        assert res.dtype == ref.dtype  # int8/int16 -> complex64, int32 -> complex128
        assert np.array_equal(res, ref)

    @pytest.mark.parametrize("size", SIZES, ids=str)
    def test_sort_complex_complex(self, size):
        a = rcomplex(np.random.default_rng(16), size)
        assert np.array_equal(num.sort_complex(a), np.sort_complex(a))


# ---- test_partition.py ----------------------------------------------------------------
def assert_partition(a, kth, axis):
    """The invariant checker of the reference: per segment, max(left) <= a[kth] <= min(right)."""
    a = np.asarray(a)
    sort_dim = a.shape[axis]
    mod = np.swapaxes(a, axis, a.ndim - 1).reshape(-1, sort_dim)
    for seg in mod:
        if kth > 0:
            assert not (seg[:kth].max() > seg[kth])
        if kth < sort_dim:
            assert not (seg[kth:].min() < seg[kth])


def assert_argpartition(idx, a_org, kth, axis):
    assert idx.dtype == np.int64
    idx_np, a_np = np.asarray(idx), np.asarray(a_org)
    assert idx_np.shape == a_np.shape
    assert_partition(np.take_along_axis(a_np, idx_np, axis=axis), kth, axis)


PARTITION_CASES = [((220,), np.uint32), ((2, 5, 7), np.int8), ((8, 5), np.float32),
                   ((2, 5, 7), np.complex128)]


class TestPartition:
    @pytest.mark.parametrize("shape, dtype", PARTITION_CASES, ids=str)
    def test_dtypes(self, shape, dtype):
        rng = np.random.default_rng(17)
        a = random_array(dtype, int(np.prod(shape)), rng, specials=False).reshape(shape)
        a_num = num.array(a)
        for axis in range(-a.ndim, a.ndim):
            for kth in (0, a.shape[axis] // 2, a.shape[axis] - 1):
                assert_partition(num.partition(a_num, kth, axis=axis), kth, axis)
                assert_argpartition(num.argpartition(a_num, kth, axis=axis), a_num, kth, axis)
                b = num.array(a)
                b.partition(kth, axis=axis)
                assert_partition(b, kth, axis)
                assert_argpartition(a_num.argpartition(kth, axis=axis), a_num, kth, axis)
        flat = num.partition(a_num, 1, axis=None)
        assert flat.shape == (a.size,)
        assert_partition(flat, 1, 0)
        assert_argpartition(num.argpartition(a_num, 1, axis=None), a.reshape(-1), 1, 0)

    @pytest.mark.parametrize("axis", (-4, 3))
    def test_axis_out_of_bound(self, axis):
        a = np.random.default_rng(18).random((3, 4, 5))
        with pytest.raises(ValueError):
            num.partition(a, kth=1, axis=axis)
        with pytest.raises(ValueError):
            num.argpartition(a, kth=1, axis=axis)

    def test_order_not_supported(self):
        with pytest.raises(NotImplementedError):
            num.partition([3, 1, 2], 1, order="x")


# ---- beyond the reference's coverage: every dtype, special floats, 4-D, tensors --------
class TestAllDtypes:
    @pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
    @pytest.mark.parametrize("shape", [(37,), (6, 40), (3, 7, 300), (2, 3, 4, 9)], ids=str)
    def test_sort_argsort_every_axis(self, dtype, shape):
        rng = np.random.default_rng(19)
        a = random_array(dtype, int(np.prod(shape)), rng).reshape(shape)
        a_num = num.array(a)
        for axis in list(range(-a.ndim, a.ndim)) + [None]:
            s = np.asarray(num.sort(a_num, axis=axis, kind="stable"))
            assert bits_equal(s, np.sort(a, axis=axis, kind="stable")), (dtype, shape, axis)
            i = np.asarray(num.argsort(a_num, axis=axis, kind="stable"))
            assert np.array_equal(i, np.argsort(a, axis=axis, kind="stable")), (dtype, shape, axis)
        assert bits_equal(np.asarray(a_num), a)  # inputs are never modified

    def test_numpy_special_float_example(self):
        a = np.array([3, np.nan, -0.0, 0.0, 1.0, -np.nan, 0.0, -0.0, -1.0], dtype=np.float32)
        assert list(np.asarray(num.argsort(a, kind="stable"))) == [8, 2, 3, 6, 7, 4, 0, 1, 5]
        assert bits_equal(np.asarray(num.sort(a)), np.sort(a, kind="stable"))

    def test_torch_tensor_input(self):
        import torch

        t = torch.randn(1000, device="cuda")
        res = num.argsort(t, kind="stable")
        assert np.array_equal(res, np.argsort(t.cpu().numpy(), kind="stable"))
        assert torch.equal(num.sort(t).to_torch(), torch.sort(t)[0])

    def test_readonly_array_cannot_sort_in_place(self):
        a = num.array([3, 1, 2])
        a.flags.writeable = False
        with pytest.raises(ValueError):
            a.sort()


# ---- shapes whose middle extent exceeds one launch dimension ---------------------------
@pytest.mark.parametrize("dtype,shape", [(np.complex128, (2, 70000, 2)), (np.float64, (600, 70000, 2))],
                         ids=["complex128", "float64"])
def test_sort_axis0_with_a_long_middle_axis(dtype, shape):
    """Sorting along axis 0 swaps it with the last axis; the planes of that copy (outer x
    middle extent) exceed the 65535 blocks a launch dimension holds."""
    rng = np.random.default_rng(91)
    a = random_array(dtype, int(np.prod(shape)), rng).reshape(shape)
    a_num = num.array(a)
    assert bits_equal(np.asarray(num.sort(a_num, axis=0)), np.sort(a, axis=0, kind="stable"))
    assert np.array_equal(np.asarray(num.argsort(a_num, axis=0, kind="stable")),
                          np.argsort(a, axis=0, kind="stable"))
