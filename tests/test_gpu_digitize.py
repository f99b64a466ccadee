"""digitize on the GPU against numpy.digitize.

Restates the reference's tests/integration/test_digitize.py: complex input and bins of two
dimensions or without an order are errors, empty input, increasing, decreasing and repeated
bin edges for uint32 / uint64 / float32 / float64 data of one to three dimensions, both
sides, array-likes and arrays mixed.  Added: many queries into many bins (the searchsorted
route that sorts the queries first), NaN and infinities."""
import numpy as np
import pytest

import cunumeric_amd as num

pytestmark = pytest.mark.gpu

DTYPES = (np.uint32, np.uint64, np.float32, np.float64)
SHAPES = ((10,), (2, 5), (3, 7, 10))


def generate_random(shape, dtype, rng):
    size = int(np.prod(shape))
    if np.issubdtype(dtype, np.integer):
        a = rng.integers(np.iinfo(dtype).min, np.iinfo(dtype).max, size=size, dtype=dtype)
    else:
        a = rng.random(size).astype(dtype)
    return a.reshape(shape)


def test_errors():
    a = np.array([2, 3, 10, 9], dtype=np.complex64)
    with pytest.raises(TypeError):
        num.digitize(a, [0, 3, 5])
    with pytest.raises(ValueError):
        num.digitize([2, 3, 10, 9], [0, 5, 3])
    with pytest.raises(ValueError):
        num.digitize([2, 3, 10, 9], np.array([[0], [5], [3]]))


@pytest.mark.parametrize("right", (True, False))
def test_empty(right):
    assert len(np.asarray(num.digitize([], [0, 3, 5], right=right))) == 0


@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("right", (True, False))
@pytest.mark.parametrize("bins", ([0, 3, 5], [10, 7, 2], [5, 3, 3, 0], [0, 3, 3, 5], [4], []), ids=str)
def test_bins(shape, dtype, right, bins):
    rng = np.random.default_rng(11)
    a = generate_random(shape, dtype, rng)
    ref = np.digitize(a, bins, right=right)
    for x, b in ((a, bins), (num.array(a), bins), (num.array(a), num.array(np.asarray(bins, dtype=np.int64)))):
        got = np.asarray(num.digitize(x, b, right=right))
        assert got.shape == ref.shape and np.array_equal(got, ref)


@pytest.mark.parametrize("right", (True, False))
def test_many_values_many_bins_and_specials(right):
    rng = np.random.default_rng(12)
    bins = np.sort(rng.standard_normal((1 << 24) + 3).astype(np.float32))     # 64 MiB of edges
    x = rng.standard_normal((1 << 20) + 5).astype(np.float32)
    x[:4] = [np.nan, np.inf, -np.inf, 0.0]
    x[4:1000] = bins[rng.integers(0, bins.size, 996)]                          # values on edges
    assert np.array_equal(np.asarray(num.digitize(x, bins, right=right)), np.digitize(x, bins, right=right))
    assert np.array_equal(np.asarray(num.digitize(x, bins[::-1].copy(), right=right)),
                          np.digitize(x, bins[::-1], right=right))
    assert int(np.asarray(num.digitize(0.5, [0.0, 1.0, 2.0], right=right))) == np.digitize(0.5, [0.0, 1.0, 2.0], right=right)
    assert int(np.asarray(num.digitize(0.5, [2.0, 1.0, 0.0], right=right))) == np.digitize(0.5, [2.0, 1.0, 0.0], right=right)
