"""Long single rows whose keys take few distinct values: the four-launch path is tried before
the radix passes (a sample with at most 255 distinct keys makes each of them a splitter with a
bin of equal keys behind it, which the scatter fills at the elements' final places), the
decision is made on the device, and the radix kernels return at once if it went through.
Exact against NumPy: values that all have bins of their own, rare values between them (sorted
by the bin sort), samples that promise more than the row keeps (the way back to the radix
path), rows with many distinct values (no attempt beyond the plan kernel), in place (no attempt
at all), a caller's payload, complex keys."""
import numpy as np
import pytest

from cunumeric_amd._lib import Options
from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu

N = (1 << 22) + 4099


@pytest.fixture(scope="module")
def abi():
    return Abi()


ON = dict(options=Options(low_cardinality=1))  # (by itself the attempt is made from 2^27 elements on)


def check(abi, a, **kw):
    n = a.size
    assert np.array_equal(abi.local_sort(a, n, argsort=True, **kw), np.argsort(a, kind="stable"))
    assert bits_equal(abi.local_sort(a, n, argsort=False, **kw), np.sort(a, kind="stable"))


def zipf_values(dtype, n, k, rng):
    dt = np.dtype(dtype)
    if dt.kind in "iu":
        ii = np.iinfo(dt)
        v = rng.integers(ii.min, ii.max, k, dtype=dt, endpoint=True)
    elif dt.kind == "f":
        v = rng.standard_normal(k).astype(dt)
        v[: min(k, 4)] = np.array([0.0, -0.0, np.nan, np.inf], dtype=dt)[: min(k, 4)]
    else:
        v = (rng.integers(-3, 3, k) + 1j * rng.integers(-3, 3, k)).astype(dt)
    w = np.arange(1, k + 1, dtype=np.float64) ** -1.2
    return v[rng.choice(k, n, p=w / w.sum())]


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32, np.int64, np.uint64, np.float64, np.complex64],
                         ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("k", [1, 2, 16, 200])
def test_few_distinct_values(abi, dtype, k):
    rng = np.random.default_rng(81)
    a = zipf_values(dtype, N, k, rng)
    plan = abi.describe_plan(dtype, N, N, True, **ON)
    print(f"low cardinality dtype={np.dtype(dtype).name} k={k} plan={plan}", flush=True)
    assert "strategy=radix" in plan and "low_cardinality_attempt=1" in plan
    assert "low_cardinality_attempt" not in abi.describe_plan(dtype, N, N, True)
    assert "low_cardinality_attempt=1" in abi.describe_plan(dtype, 1 << 27, 1 << 27, True)
    check(abi, a, **ON)


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float64], ids=lambda d: np.dtype(d).name)
def test_rare_values_between_the_common_ones(abi, dtype):
    """250 common values and one element in a hundred drawn from the whole range: the rare
    ones land in the bins between the splitters and are sorted there."""
    rng = np.random.default_rng(82)
    a = zipf_values(dtype, N, 250, rng)
    rare = rng.random(N) < 0.01
    a[rare] = random_array(dtype, int(rare.sum()), rng, specials=False)
    check(abi, a, **ON)
    pay = rng.integers(-2**62, 2**62, N, dtype=np.int64)
    got = abi.local_sort(a, N, argsort=True, indices_in=pay, **ON)
    assert np.array_equal(got, pay[np.argsort(a, kind="stable")])
    got = abi.local_sort(a, N, argsort=True, index_offset=-77, **ON)
    assert np.array_equal(got, np.argsort(a, kind="stable") - 77)


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64, np.complex64], ids=lambda d: np.dtype(d).name)
def test_way_back_to_the_radix_path(abi, dtype):
    """low_cardinality = 2 tries with any sample.  Random keys: the bins between the splitters
    are far longer than the bin sort holds, the scatter says so and the radix kernels run.
    Also the sample's blind spot: a value that fills a third of the row's tail but sits between
    the sample's places is found by the count, not by the sample."""
    rng = np.random.default_rng(83)
    a = random_array(dtype, N, rng)
    check(abi, a, options=Options(low_cardinality=2))
    check(abi, a, **ON)  # the plan kernel alone sees that the values are many
    check(abi, a, options=Options(low_cardinality=0))
    b = zipf_values(dtype, N, 12, rng)
    b[rng.integers(0, N, N // 50)] = random_array(dtype, N // 50, rng, specials=False)[0]
    idx = rng.integers(0, N, 300000)
    b[idx] = random_array(dtype, idx.size, rng, specials=False)  # many rare values: bins too long
    check(abi, b, **ON)
    check(abi, b, options=Options(low_cardinality=2))


def test_in_place_keeps_the_radix_path(abi):
    rng = np.random.default_rng(84)
    a = zipf_values(np.int64, N, 16, rng)
    assert bits_equal(abi.local_sort(a, N, argsort=False, inplace=True, **ON), np.sort(a, kind="stable"))
    pay = rng.integers(-2**62, 2**62, N, dtype=np.int64)
    got = abi.local_sort(a, N, argsort=True, indices_in=pay, inplace=True, **ON)
    assert np.array_equal(got, pay[np.argsort(a, kind="stable")])


def test_unique_and_python_surface(abi):
    """2^27 elements: the built-in plan makes the attempt."""
    import cunumeric_amd as num

    rng = np.random.default_rng(85)
    a = zipf_values(np.int32, 1 << 27, 40, rng)
    assert np.array_equal(np.asarray(num.unique(num.array(a))), np.unique(a))
    assert np.array_equal(np.asarray(num.argsort(num.array(a), kind="stable")), np.argsort(a, kind="stable"))
    assert np.array_equal(np.asarray(num.sort(num.array(a))), np.sort(a))
