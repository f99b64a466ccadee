"""quantile / percentile on the GPU against numpy.quantile / numpy.percentile.

Restates the reference's tests/integration/test_quantiles.py and test_percentiles.py: all 13
methods x single and several axes x scalar and array q x keepdims x overwrite_input, an output
array, axis=None, q = 0 and 1, array-likes as input, the output dtype rule; NumPy is the
oracle, as it is there (tolerance 1e-8 as in the reference; the sample-returning methods are
compared exactly).  Added: long rows, which take the selection path, and NaNs."""
import numpy as np
import pytest

import cunumeric_amd as num
from cunumeric_amd.quantile import METHODS

pytestmark = pytest.mark.gpu

EPS = 1.0e-8
QS = [0.001, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49, 0.5]
SAMPLE_METHODS = ("inverted_cdf", "closest_observation", "lower", "higher", "nearest")


def check(got, ref, method, in_dtype=None):
    got = np.asarray(got)
    assert got.shape == np.shape(ref)
    if in_dtype is not None and method not in SAMPLE_METHODS:
        # the reference's rule (cunumeric/module.py:8480-8511): float64 unless the method returns
        # a sample; NumPy 2 keeps float32 for float32 input, the reference does not
        assert got.dtype == np.float64
    else:
        assert got.dtype == np.asarray(ref).dtype
    if method in SAMPLE_METHODS:
        assert np.array_equal(got, ref, equal_nan=True)
    else:
        assert np.allclose(got, ref, atol=EPS, rtol=0, equal_nan=True)


def small_3d():
    return np.array([1, 2, 2, 40, 1, 1, 2, 1, 0, 10, 3, 3, 40, 15, 3, 7, 5, 4, 7, 3, 5, 1, 0, 9],
                    dtype=int).reshape(2, 3, 4)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (0, 1, (0, 1), (0, 2)))
@pytest.mark.parametrize("qin", (0.5, QS))
@pytest.mark.parametrize("keepdims", (False, True))
@pytest.mark.parametrize("overwrite_input", (False, True))
def test_multi_axes(method, axes, qin, keepdims, overwrite_input):
    arr = small_3d()
    q = qin if np.isscalar(qin) else np.array(qin)
    got = num.quantile(num.array(arr), q, axis=axes, method=method, keepdims=keepdims,
                       overwrite_input=overwrite_input)
    ref = np.quantile(arr.copy(), q, axis=axes, method=method, keepdims=keepdims)
    check(got, ref, method)
    gotp = num.percentile(num.array(arr), np.asarray(q) * 100.0, axis=axes, method=method, keepdims=keepdims)
    check(gotp, np.percentile(arr, np.asarray(q) * 100.0, axis=axes, method=method, keepdims=keepdims), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("ls_in", ([[1.0, 0.13, 2.11], [1.9, 9.2, 0.17]],
                                   [[1, 1, 0], [2, 1, 10], [2, 2, 3], [40, 1, 3], [40, 5, 5], [15, 4, 1],
                                    [3, 7, 0], [7, 3, 9]]))
@pytest.mark.parametrize("axes", (0, 1))
@pytest.mark.parametrize("keepdims", (False, True))
def test_nd_quantile(method, ls_in, axes, keepdims):
    arr = np.array(ls_in)
    q = np.array([[0.001, 0.37, 0.42], [0.67, 0.83, 0.99]])
    check(num.quantile(arr, q, axis=axes, method=method, keepdims=keepdims),
          np.quantile(arr, q, axis=axes, method=method, keepdims=keepdims), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (0, 1))
@pytest.mark.parametrize("qs", (0.5, np.array([0.001, 0.37, 0.42, 0.67])))
@pytest.mark.parametrize("keepdims", (False, True))
def test_quantiles_with_output(method, axes, qs, keepdims):
    arr = np.array([[1, 1, 0], [2, 1, 10], [2, 2, 3], [40, 1, 3], [40, 5, 5], [15, 4, 1], [3, 7, 0],
                    [7, 3, 9]])
    ref = np.quantile(arr, qs, axis=axes, method=method, keepdims=keepdims)
    out = num.array(np.zeros(ref.shape, dtype=np.float64))
    res = num.quantile(arr, qs, axis=axes, out=out, method=method, keepdims=keepdims)
    assert res is out
    assert np.allclose(np.asarray(out), ref, atol=EPS)
    with pytest.raises(ValueError):
        num.quantile(arr, qs, axis=axes, out=num.array(np.zeros((7, 7, 7))), method=method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("qin", (0.5, QS))
@pytest.mark.parametrize("keepdims", (False, True))
def test_quantiles_axis_none(method, qin, keepdims):
    arr = small_3d()
    q = qin if np.isscalar(qin) else np.array(qin)
    check(num.quantile(arr, q, method=method, keepdims=keepdims),
          np.quantile(arr, q, method=method, keepdims=keepdims), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (None, 0))
def test_random(method, axes):
    rng = np.random.default_rng(17)
    arr = rng.random((3, 4, 5))
    q = rng.random(7)
    check(num.quantile(arr, q, axis=axes, method=method), np.quantile(arr, q, axis=axes, method=method), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("q", (0.0, 1.0))
def test_quantile_at_the_ends(method, q):
    arr = np.arange(24, dtype=np.float64).reshape(2, 3, 4)
    check(num.quantile(arr, q, axis=0, method=method), np.quantile(arr, q, axis=0, method=method), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("arr", (3, (3,), [3], (2, 1), [2, 1]))
def test_non_ndarray_input(method, arr):
    q = np.array([0.001, 0.37, 0.42, 0.67])
    check(num.quantile(arr, q, method=method), np.quantile(arr, q, method=method), method)


def test_output_dtype_rule_and_errors():
    arr = np.array([[1, 2, 7], [5, 3, 1]], dtype=np.int16)
    for method in METHODS:
        got = num.quantile(arr, 0.3, axis=1, method=method)
        assert got.dtype == np.quantile(arr, 0.3, axis=1, method=method).dtype
    with pytest.raises(TypeError):
        num.quantile(np.array([1 + 2j, 3 - 1j]), 0.5)
    with pytest.raises(ValueError):
        num.quantile(arr, 0.5, method="median")
    with pytest.raises(ValueError):
        num.quantile(arr, 1.5)
    with pytest.raises(ValueError):
        num.percentile(arr, 101)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64, np.uint32, np.uint64])
@pytest.mark.parametrize("method", ("linear", "hazen", "lower", "nearest", "averaged_inverted_cdf"))
def test_long_rows_take_the_selection_path(dtype, method):
    """One quantile of long rows: found by radix select (no row is sorted or moved)."""
    rng = np.random.default_rng(23)
    n = (1 << 17) + 77
    if np.dtype(dtype).kind == "f":
        a = rng.standard_normal((3, n)).astype(dtype)
    elif np.dtype(dtype).kind == "u":
        a = rng.integers(0, 2000, (3, n)).astype(dtype)
    else:
        a = rng.integers(-1000, 1000, (3, n)).astype(dtype)
    a64 = a.astype(np.float64) if np.dtype(dtype) == np.float32 else a  # NumPy blends in the input's precision
    for q in (0.5, 0.013, 1.0):
        check(num.quantile(a, q, axis=1, method=method), np.quantile(a64, q, axis=1, method=method).astype(
            a.dtype if method in SAMPLE_METHODS else np.float64), method, a.dtype)
    check(num.quantile(a, 0.25, method=method),
          np.quantile(a64, 0.25, method=method).astype(a.dtype if method in SAMPLE_METHODS else np.float64),
          method, a.dtype)
    check(num.percentile(a, [10.0, 50.0, 90.0], axis=1, method=method),
          np.percentile(a64, [10.0, 50.0, 90.0], axis=1, method=method).astype(
              a.dtype if method in SAMPLE_METHODS else np.float64), method, a.dtype)


def test_rows_with_nan_have_no_quantile():
    a = np.random.default_rng(3).standard_normal((4, 1000))
    a[1, 17] = np.nan
    a[3, 999] = np.nan
    for method in ("linear", "lower", "midpoint"):
        check(num.quantile(a, [0.1, 0.9], axis=1, method=method),
              np.quantile(a, [0.1, 0.9], axis=1, method=method), method)
    # long rows (the selection path): the largest element of a row tells the NaN
    b = np.random.default_rng(4).standard_normal((3, 70001))
    b[2, 5] = np.nan
    for method in ("linear", "lower", "midpoint"):
        for q in (0.5, 0.999):
            check(num.quantile(b, q, axis=1, method=method), np.quantile(b, q, axis=1, method=method), method)
