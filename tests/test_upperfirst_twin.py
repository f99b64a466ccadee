"""The rules of the sort of 8-byte keys by their upper bytes first, on the CPU: the number of
upper bytes against what the library plans (its plan description names it), and the fix-up's
rules against a full stable sort.  No GPU."""
import numpy as np
import pytest

from cunumeric_amd import _lib
from cunumeric_amd._lib import Options
from tests import upperfirst_twin as tw


@pytest.mark.parametrize("code,kind", [(4, "i"), (8, "i"), (11, "f"), (12, "c")])
def test_upper_bytes_kept_match_the_library(code, kind):
    o = Options(bucket_path=0, upper_first=1)
    for lg in range(15, 34):
        for row_len in ((1 << lg) - 1, 1 << lg, (1 << lg) + 1, 3 << (lg - 1)):
            plan = _lib.describe_plan(code, row_len, row_len, True, options=o)
            assert f"upper_digits={8 - tw.digit0(kind, row_len)} " in plan + " ", (row_len, plan)
    # expected run length at most 1/32 with keys spread evenly over the bits that tell values
    # apart, unless six bytes (the most the attempt keeps) are not enough for that
    spent = {"i": 0, "f": 12, "c": 15}[kind]
    for lg in range(15, 40):
        nbytes = 8 - tw.digit0(kind, 1 << lg)
        assert 4 <= nbytes <= 6
        assert 8 * nbytes - spent >= lg + 5 or nbytes == 6
        assert nbytes == 4 or 8 * (nbytes - 1) - spent < lg + 5   # (and no byte more than needed)


def upper_sorted(keys, low_bits):
    order = np.argsort(keys >> np.uint64(low_bits), kind="stable")
    return keys[order], order.astype(np.int64)


@pytest.mark.parametrize("low_bits", [16, 24, 32])
@pytest.mark.parametrize("mean_run", [1.0, 1.5, 4.0, 12.0, 40.0])
def test_fix_up_rules_give_the_stable_sort_or_call_the_attempt_off(low_bits, mean_run):
    rng = np.random.default_rng(int(low_bits * 100 + mean_run * 10))
    for trial in range(6):
        n = int(rng.integers(1000, 20000))
        lengths = rng.geometric(1.0 / mean_run, n)
        upper = np.repeat(rng.permutation(lengths.size).astype(np.uint64), lengths)[:n]
        low = rng.integers(0, 1 << int(rng.integers(1, low_bits + 1)), n).astype(np.uint64)
        keys = ((upper << np.uint64(low_bits)) | low)[rng.permutation(n)]
        k1, p1 = upper_sorted(keys, low_bits)
        k2, p2, done = tw.fixup(k1, p1, low_bits)
        want = np.argsort(keys, kind="stable")
        if done:
            assert np.array_equal(p2, want) and np.array_equal(k2, keys[want])
        else:
            # only a run beyond the limit that holds an element out of order calls it off
            up = k1 >> np.uint64(low_bits)
            starts = np.flatnonzero(np.concatenate([[True], up[1:] != up[:-1]]))
            ends = np.concatenate([starts[1:], [n]])
            assert any(e - s > tw.RUN_LIMIT and np.any(k1[s:e][:-1] > k1[s:e][1:]) for s, e in zip(starts, ends))


def test_runs_of_equal_keys_of_any_length_do_not_call_it_off():
    rng = np.random.default_rng(5)
    pool = rng.integers(0, 1 << 63, 50, dtype=np.uint64)
    keys = pool[rng.integers(0, 50, 30000)]
    k1, p1 = upper_sorted(keys, 24)
    k2, p2, done = tw.fixup(k1, p1, 24)
    assert done and np.array_equal(p2, np.argsort(keys, kind="stable"))
