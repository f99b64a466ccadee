"""Where a quantile lies in a sorted sample (cunumeric_amd.quantile._position) against
numpy.quantile for all 13 methods: the blend of the two named samples must reproduce NumPy on
sorted data of many lengths, including quantiles that fall exactly on samples, q = 0 and 1.
No GPU: only the host arithmetic is exercised."""
import numpy as np
import pytest

from cunumeric_amd.quantile import METHODS, _position


def blend(x, lo, hi, g):
    if lo == hi or g == 0.0:
        return float(x[lo])
    d = float(x[hi]) - float(x[lo])
    return float(x[lo]) + d * g if g < 0.5 else float(x[hi]) - d * (1.0 - g)


@pytest.mark.parametrize("method", METHODS)
def test_position_matches_numpy(method):
    rng = np.random.default_rng(3)
    qs = [0.0, 1.0, 0.5, 0.25, 0.75, 1 / 3, 2 / 3, 0.001, 0.999, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49]
    for n in (1, 2, 3, 4, 5, 7, 8, 10, 11, 16, 33, 100, 101):
        x = np.sort(rng.standard_normal(n))
        for q in qs + [k / n for k in range(n + 1)] + [(k + 0.5) / n for k in range(n)]:
            lo, hi, g = _position(method, float(q), n)
            assert 0 <= lo <= hi < n
            ref = float(np.quantile(x, q, method=method))
            assert blend(x, lo, hi, g) == pytest.approx(ref, rel=1e-13, abs=1e-13), (n, q)


def test_unknown_method():
    with pytest.raises(ValueError):
        _position("median", 0.5, 10)


@pytest.mark.parametrize("method", METHODS)
def test_positions_of_many_sample_sizes_at_once(method):
    """The tensor form used by nanquantile (every slice has its own number of non-NaN
    elements) names the same two samples and weight as the scalar form."""
    import torch

    from cunumeric_amd.quantile import _position_rows

    sizes = list(range(1, 70)) + [100, 101, 1000, 4097]
    n = torch.tensor(sizes, dtype=torch.int64)
    for q in [0.0, 1.0, 0.5, 0.25, 0.75, 1 / 3, 2 / 3, 0.001, 0.999, 0.37, 0.42, 0.67, 0.83, 0.99, 0.39, 0.49,
              0.1, 0.2, 0.3, 0.6]:
        lo, hi, g = _position_rows(method, q, n)
        for k, size in enumerate(sizes):
            a, b, w = _position(method, q, size)
            assert (int(lo[k]), int(hi[k])) == (a, b) or (w == 0.0 and float(g[k]) == 0.0 and int(lo[k]) == a), (q, size)
            assert float(g[k]) == pytest.approx(w, abs=1e-12), (q, size)
