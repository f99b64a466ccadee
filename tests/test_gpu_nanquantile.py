"""nanquantile / nanpercentile on the GPU against numpy.nanquantile / numpy.nanpercentile.

Restates the reference's tests/integration/test_nanquantiles.py and test_nanpercentiles.py
(all 13 methods x both axes x scalar and array q on a (3, 4) array with NaNs, tolerance 1e-8;
NumPy is the oracle, as it is there).  Added: several axes, axis=None, keepdims, an output
array, slices of NaNs only, input without NaNs (must equal quantile), float32 and integer
input, rows long enough for the radix path."""
import warnings

import numpy as np
import pytest

import cunumeric_amd as num
from cunumeric_amd.quantile import METHODS

pytestmark = pytest.mark.gpu

EPS = 1.0e-8
QS = [0.001, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49, 0.5]
SAMPLE_METHODS = ("inverted_cdf", "closest_observation", "lower", "higher", "nearest")


def check(got, ref, method):
    got = np.asarray(got)
    assert got.shape == np.shape(ref)
    if method in SAMPLE_METHODS:
        assert got.dtype == np.asarray(ref).dtype
        assert np.array_equal(got, ref, equal_nan=True)
    else:
        assert got.dtype == np.float64   # the reference's rule (cunumeric/module.py:8916-8932)
        assert np.allclose(got, ref, atol=EPS, rtol=0, equal_nan=True)


def nan_3x4():
    return np.ndarray(shape=(3, 4), buffer=np.array([1.0, 2, 2, 40, 1, np.nan, 2, 1, 0, 10, np.nan, np.nan]),
                      dtype=float)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (0, 1))
@pytest.mark.parametrize("qin", (0.5, QS))
def test_multi_axes(method, axes, qin):
    arr = nan_3x4()
    q = qin if np.isscalar(qin) else np.array(qin)
    got = num.nanquantile(num.array(arr), q, axis=axes, method=method, keepdims=False, overwrite_input=False)
    check(got, np.nanquantile(arr, q, axis=axes, method=method, keepdims=False), method)
    gotp = num.nanpercentile(num.array(arr), np.asarray(q) * 100.0, axis=axes, method=method)
    check(gotp, np.nanpercentile(arr, np.asarray(q) * 100.0, axis=axes, method=method), method)


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("axes", (None, (0, 1), (0, 2), 2, -1))
@pytest.mark.parametrize("keepdims", (False, True))
def test_more_axes_keepdims(method, axes, keepdims):
    rng = np.random.default_rng(5)
    arr = rng.standard_normal((4, 3, 5))
    arr[rng.random(arr.shape) < 0.3] = np.nan
    arr[1, 2, :] = np.nan                      # a slice of NaNs only along the last axis
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)   # NumPy: "All-NaN slice encountered"
        ref = np.nanquantile(arr, QS, axis=axes, method=method, keepdims=keepdims)
    check(num.nanquantile(arr, QS, axis=axes, method=method, keepdims=keepdims), ref, method)


@pytest.mark.parametrize("method", ("linear", "hazen", "lower", "nearest", "inverted_cdf"))
def test_without_nans_equals_quantile_and_dtypes(method):
    rng = np.random.default_rng(6)
    for dtype in (np.float64, np.float32, np.int32, np.int64):
        arr = (rng.standard_normal((7, 9)) * 50).astype(dtype)
        a = np.asarray(num.nanquantile(arr, [0.1, 0.5, 0.9], axis=1, method=method))
        b = np.asarray(num.quantile(arr, [0.1, 0.5, 0.9], axis=1, method=method))
        assert a.dtype == b.dtype and np.array_equal(a, b)
        ref = np.nanquantile(arr.astype(np.float64) if method not in SAMPLE_METHODS else arr, [0.1, 0.5, 0.9],
                             axis=1, method=method)
        assert np.allclose(a, ref, atol=EPS, rtol=0)


def test_output_array_errors_and_long_rows():
    rng = np.random.default_rng(7)
    arr = rng.standard_normal((3, 70001)).astype(np.float32)     # rows on the radix path
    arr[rng.random(arr.shape) < 0.1] = np.nan
    arr[2, 5:] = np.nan                                          # five elements left
    ref = np.nanquantile(arr.astype(np.float64), [0.25, 0.5], axis=1)
    got = num.nanquantile(arr, [0.25, 0.5], axis=1)
    assert np.allclose(np.asarray(got), ref, atol=1e-6, rtol=0)
    out = num.array(np.zeros((2, 3)))
    res = num.nanquantile(arr, [0.25, 0.5], axis=1, out=out)
    assert res is out and np.allclose(np.asarray(out), ref, atol=1e-6, rtol=0)
    with pytest.raises(ValueError):
        num.nanquantile(arr, [0.25, 0.5], axis=1, out=num.array(np.zeros((3, 2))))
    with pytest.raises(TypeError):
        num.nanquantile(np.array([1 + 2j, 3 + 1j]), 0.5)
    with pytest.raises(ValueError):
        num.nanquantile(arr, 1.5)
    with pytest.raises(ValueError):
        num.nanpercentile(arr, 101)
    with pytest.raises(ValueError):
        num.nanquantile(arr, 0.5, method="median")
    # scalar q, axis None
    got = num.nanquantile(arr, 0.5)
    assert np.asarray(got).shape == () and np.isclose(float(np.asarray(got)), np.nanquantile(arr.astype(np.float64), 0.5),
                                                      atol=1e-6)
