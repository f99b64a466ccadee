"""The index logic of the four-launch sort of medium rows (cunumeric_amd/csrc/bucket.hpp),
restated on the CPU in tests/bucket_twin.py, against numpy's stable argsort: search tree and
bins, sample places, scatter offsets, and the claim that keys between two splitters differ
only below the splitters' common prefix."""
import numpy as np
import pytest

from tests import bucket_twin as tw


def test_tree_search_counts_the_splitters_below_a_key():
    rng = np.random.default_rng(1)
    for dtype in (np.uint8, np.uint16, np.uint32, np.uint64):
        top = np.iinfo(dtype).max
        for m in (1, 2, 17, 255):
            spl = np.full(tw.SLOTS, top, dtype=dtype)
            spl[:m] = np.sort(rng.integers(0, top, m, dtype=dtype, endpoint=True))
            tree = tw.tree_of(spl)
            keys = np.concatenate([rng.integers(0, top, 5000, dtype=dtype, endpoint=True), spl,
                                   np.array([0, top], dtype=dtype)])
            got = tw.bin_of(spl, tree, keys)
            below = np.searchsorted(spl[:255], keys, side="left")  # splitters strictly below
            equal = spl[below] == keys
            assert np.array_equal(got, 2 * below + equal)
            assert got.max() < tw.BINS


def test_sample_places_stay_inside_their_stretch():
    for n, m in ((16385, 16), (100003, 97), (1 << 20, 255), (300, 255)):
        pos = tw.sample_places(n, m)
        assert pos.min() >= 0 and pos.max() < n
        s = (m + 1) * tw.OVERSAMPLE
        if n >= s:
            lo = np.arange(s) * n // s
            assert np.all(pos >= lo) and np.all(pos <= lo + n // s)


@pytest.mark.parametrize("case", ["uniform32", "uniform64", "small_range", "two_values", "constant", "sorted",
                                  "sawtooth", "skewed", "top_keys", "u8", "u16", "clusters64", "low_bits64"])
def test_twin_sorts_like_a_stable_argsort(case):
    rng = np.random.default_rng(hash(case) % 1000)
    n = 50021
    if case == "uniform32":
        k = rng.integers(0, 2**32, n, dtype=np.uint32)
    elif case == "uniform64":
        k = rng.integers(0, 2**64, n, dtype=np.uint64)
    elif case == "small_range":
        k = rng.integers(0, 1000, n, dtype=np.uint64) + np.uint64(2**63)
    elif case == "two_values":
        k = rng.integers(0, 2, n, dtype=np.uint32) * np.uint32(77777)
    elif case == "constant":
        k = np.full(n, 0xDEADBEEF, dtype=np.uint32)
    elif case == "sorted":
        k = np.sort(rng.integers(0, 2**32, n, dtype=np.uint32))
    elif case == "sawtooth":
        k = (np.arange(n, dtype=np.uint32) % np.uint32(3126)) * np.uint32(1000003)
    elif case == "skewed":
        k = np.minimum(np.exp(rng.standard_normal(n) * 8 + 20), 1e19).astype(np.uint64)
    elif case == "top_keys":
        k = np.where(rng.random(n) < 0.3, np.uint32(0xFFFFFFFF), rng.integers(0, 2**32, n, dtype=np.uint32))
        k = k.astype(np.uint32)
    elif case == "clusters64":   # neighbours that agree in the upper bits and differ below: all passes
        far = np.array([0, 1 << 62, (1 << 62) + (1 << 45)], dtype=np.uint64)
        k = far[rng.integers(0, 3, n)] + rng.integers(0, 1 << 20, n, dtype=np.uint64)
    elif case == "low_bits64":   # a few huge keys stretch the bins' bounds; the rest differs low down
        k = rng.integers(0, 1 << 12, n, dtype=np.uint64)
        k[rng.integers(0, n, 40)] = rng.integers(1 << 50, 1 << 63, 40, dtype=np.uint64)
    elif case == "u8":
        k = rng.integers(0, 256, n, dtype=np.uint8)
    else:
        k = rng.integers(0, 65536, n, dtype=np.uint16)
    for n_split in (1, 12, 48, 255):
        order, bins = tw.bucket_argsort(k, n_split)
        assert np.array_equal(order, np.argsort(k, kind="stable")), (case, n_split)


def test_upper_bits_first_rule():
    assert [tw.upper_bits_first(b) for b in (1, 40, 41, 47, 48, 55, 56, 57, 64)] == [0, 0, 0, 0, 8, 8, 16, 16, 24]
    rng = np.random.default_rng(3)
    sub = rng.integers(0, 1 << 20, 5000, dtype=np.uint64) + (rng.integers(0, 2, 5000, dtype=np.uint64) << np.uint64(60))
    assert np.array_equal(tw.sort_bin(sub, 61, True), np.argsort(sub, kind="stable"))   # falls back to all bits
    sub = rng.integers(0, 1 << 61, 5000, dtype=np.uint64)
    assert np.array_equal(tw.sort_bin(sub, 61, True), np.argsort(sub, kind="stable"))   # upper bits suffice
