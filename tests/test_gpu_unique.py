"""unique on the GPU against numpy.unique.

Restates the reference's integration test (tests/integration/test_unique.py:24-71: 0 to 4
dimensions of small integers, the result of another operation as input, keyword arguments
rejected) and adds every dtype, ties, special floating-point values and sizes across the
sort strategies."""
import numpy as np
import pytest

import cunumeric_amd as num
from tests.util import ALL_DTYPES, random_array

pytestmark = pytest.mark.gpu


def same_values(got, ref):
    """equal element by element, all NaNs alike (which NaN pattern survives is not
    defined: numpy keeps whichever its unstable sort put first)"""
    got, ref = np.asarray(got), np.asarray(ref)
    return got.shape == ref.shape and got.dtype == ref.dtype and np.array_equal(got, ref, equal_nan=True)


def reference_unique(a):
    """numpy.unique, except for float16: numpy.unique sorts with the default kind, which
    returns unsorted (and so not unique) output for float16 on this x86 host (NumPy 2.2),
    so the same definition is spelled out over the stable sort."""
    a = np.asarray(a)
    if a.dtype != np.float16:
        return np.unique(a)
    s = np.sort(a.reshape(-1), kind="stable")
    nan = np.isnan(s)
    body = s[~nan]
    keep = np.ones(body.shape, dtype=bool)
    keep[1:] = body[1:] != body[:-1]
    return np.concatenate([body[keep], s[nan][:1]])


@pytest.mark.parametrize("ndim", range(5))
def test_ndim(ndim):
    rng = np.random.default_rng(ndim)
    a = rng.integers(0, 3, size=(4,) * ndim)
    assert same_values(num.unique(a), np.unique(a))
    assert same_values(num.array(a).unique(), np.unique(a))


def test_small_and_empty():
    assert same_values(num.unique(np.array([0, 1], dtype=np.int64)), np.array([0, 1]))
    assert same_values(num.unique(np.array([], dtype=np.float32)), np.array([], dtype=np.float32))
    assert same_values(num.unique(np.array([5.0])), np.array([5.0]))
    assert same_values(num.unique(np.zeros(1000, dtype=np.int8)), np.zeros(1, dtype=np.int8))


@pytest.mark.parametrize("kw", [dict(return_index=True), dict(return_inverse=True),
                                dict(return_counts=True), dict(axis=1)])
def test_keyword_arguments_rejected(kw):
    with pytest.raises(NotImplementedError):
        num.unique(np.arange(9).reshape(3, 3), **kw)


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
def test_all_dtypes(dtype):
    rng = np.random.default_rng(41)
    for n, narrow in ((1, False), (300, True), (5000, False), (5000, True), (100003, True),
                      (100003, False), ((1 << 20) + 5, True)):
        a = random_array(dtype, n, rng, narrow=narrow)
        print(f"unique dtype={np.dtype(dtype).name} n={n} narrow={narrow}", flush=True)
        assert same_values(num.unique(a), reference_unique(a)), (dtype, n, narrow)


def test_signed_zeros_and_nans_collapse():
    a = np.array([0.0, -0.0, np.nan, 1.0, -np.nan, -0.0, 1.0, np.inf, -np.inf], dtype=np.float32)
    got = np.asarray(num.unique(a))
    assert got.shape == (5,) and np.isnan(got[-1]) and got[0] == -np.inf and got[1] == 0.0
    c = np.array([1 + 2j, complex(np.nan, 1), complex(2, np.nan), 1 + 2j, complex(np.nan, np.nan)],
                 dtype=np.complex64)
    got = np.asarray(num.unique(c))
    assert got.shape == (2,) and got[0] == 1 + 2j and np.isnan(got[1])
    assert same_values(got, np.unique(c))


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.float32, np.int64, np.complex128],
                         ids=lambda d: np.dtype(d).name)
def test_sizes_around_the_compaction_blocks(dtype):
    """The compaction works on blocks of 64 KB with a vector path for whole blocks."""
    rng = np.random.default_rng(43)
    blk = 65536 // np.dtype(dtype).itemsize
    for n in (blk - 1, blk, blk + 1, 2 * blk, 3 * blk + 5):
        for narrow in (False, True):
            a = random_array(dtype, n, rng, narrow=narrow)
            print(f"unique dtype={np.dtype(dtype).name} n={n} narrow={narrow}", flush=True)
            assert same_values(num.unique(a), reference_unique(a)), (dtype, n, narrow)


def test_abi_empty_input_writes_only_the_counter():
    """misort_unique with volume 0 stores the 8-byte count and nothing beyond it."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    guard = torch.full((4,), 0x5A5A5A5A5A5A5A5A, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.misort_unique(to_core_dtype(np.dtype(np.int32)), None, None, guard.data_ptr() + 8, 0, None, 0,
                           stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert guard.cpu().tolist() == [0x5A5A5A5A5A5A5A5A, 0, 0x5A5A5A5A5A5A5A5A, 0x5A5A5A5A5A5A5A5A]
    # a misaligned counter is refused before anything is written
    assert lib.misort_unique(to_core_dtype(np.dtype(np.int32)), None, None, guard.data_ptr() + 4, 0, None,
                             0, stream) == 5
