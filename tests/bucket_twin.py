"""CPU restatement of the index logic of cunumeric_amd/csrc/bucket.hpp, element by element
where the kernels go thread by thread: the search tree over the splitters and the bin of a
key (load_splitters, bin_of), the sample places of the plan kernel (sort_sample), the offsets
of the scatter (chunks in order inside every bin) and the bits a bin sort has to look at
(the common prefix of the two splitters around the bin).  Every index is bounds-checked by
NumPy; the result is compared with a stable sort by the caller."""
from __future__ import annotations

import numpy as np

SLOTS, BINS, OVERSAMPLE = 256, 512, 16


def tree_of(sorted_spl: np.ndarray) -> np.ndarray:
    """load_splitters: node j (1..255) of the complete tree over sorted[0..254]."""
    assert sorted_spl.shape == (SLOTS,)
    tree = np.empty(SLOTS, dtype=sorted_spl.dtype)
    tree[0] = sorted_spl[0]
    for j in range(1, SLOTS):
        level = j.bit_length() - 1
        pos = j - (1 << level)
        tree[j] = sorted_spl[((2 * pos + 1) << (7 - level)) - 1]
    return tree


def bin_of(sorted_spl: np.ndarray, tree: np.ndarray, keys: np.ndarray) -> np.ndarray:
    j = np.ones(keys.shape, dtype=np.int64)
    for _ in range(8):
        j = 2 * j + (keys > tree[j])
    j -= SLOTS
    assert j.min(initial=0) >= 0 and j.max(initial=0) <= 255
    return 2 * j + (sorted_spl[j] == keys)


def sample_places(n: int, n_split: int, oversample: int = OVERSAMPLE) -> np.ndarray:
    s = (n_split + 1) * oversample
    e = np.arange(s, dtype=np.uint64)
    h = (e * np.uint64(0x9E3779B1)) & np.uint64(0xFFFFFFFF)
    h ^= h >> np.uint64(15)
    h = (h * np.uint64(0x85EBCA77)) & np.uint64(0xFFFFFFFF)
    h ^= h >> np.uint64(13)
    span = max(n // s, 1)
    pos = e * np.uint64(n) // np.uint64(s) + h % np.uint64(span)
    return np.minimum(pos, np.uint64(n - 1)).astype(np.int64)


def splitters_of(keys: np.ndarray, n_split: int) -> np.ndarray:
    """bucket_plan_kernel: every 16th key of the sorted sample, padded with the largest key."""
    sample = np.sort(keys[sample_places(keys.size, n_split)])
    spl = np.full(SLOTS, np.iinfo(keys.dtype).max, dtype=keys.dtype)
    spl[:n_split] = sample[OVERSAMPLE - 1::OVERSAMPLE][:n_split]
    return spl


def bin_bits(spl: np.ndarray, g: int, kmin: int = 0, kmax: int | None = None):
    """bucket_sort_kernel: keys strictly between splitters g-1 and g are sorted by key - lo,
    which has at most as many bits as hi - lo; the first bin starts at the row's smallest key
    and no bin reaches beyond its largest (count kernel -> chunk 0 of the scatter)."""
    lo = int(spl[g - 1]) if g > 0 else int(kmin)
    hi = int(spl[g]) if kmax is None else min(int(spl[g]), int(kmax))
    return lo, (hi - lo).bit_length()


def upper_bits_first(nbits: int) -> int:
    """8-byte keys: the first bit of the 40 to 47 upper ones of [0, nbits) that the bin sort
    looks at first (0: all of them anyway)."""
    hb = nbits - 1
    if hb < 40:
        return 0
    return 8 * ((hb + 1 - 40) // 8)


def sort_bin(sub: np.ndarray, nbits: int, eight_byte: bool) -> np.ndarray:
    """Order of a bin by its reduced keys the way block_radix_sort_rows gets there: by the upper
    bits first; if two neighbours of that order agree in them and differ below, by all bits
    from that order on (stable passes: equal keys never trade places)."""
    lo = upper_bits_first(nbits) if eight_byte else 0
    if lo == 0:
        return np.argsort(sub, kind="stable")
    first = np.argsort(sub >> np.uint64(lo), kind="stable")
    s = sub[first]
    bad = np.any(((s[1:] >> np.uint64(lo)) == (s[:-1] >> np.uint64(lo))) & (s[1:] != s[:-1]))
    return first[np.argsort(s, kind="stable")] if bad else first


def bucket_argsort(keys: np.ndarray, n_split: int, tile: int = 4096, chunks_per_slab: int = 16):
    """Stable argsort of unsigned keys the way the four kernels do it; returns (order, bins)."""
    n = keys.size
    spl = splitters_of(keys, n_split)
    assert np.all(spl[:-1] <= spl[1:])
    tree = tree_of(spl)
    bins = bin_of(spl, tree, keys)
    # count kernel: per chunk and bin; scatter prologue: bins before, slabs before, chunks before
    tiles = -(-n // tile)
    want = min(tiles, 256)
    tpc = -(-tiles // want)
    n_chunks = -(-tiles // tpc)
    clen = tpc * tile
    chunk_hist = np.zeros((n_chunks, BINS), dtype=np.int64)
    for c in range(n_chunks):
        chunk_hist[c] = np.bincount(bins[c * clen:(c + 1) * clen], minlength=BINS)
    n_slabs = -(-n_chunks // chunks_per_slab)
    slab_tot = np.zeros((n_slabs, BINS), dtype=np.int64)
    for c in range(n_chunks):
        slab_tot[c // chunks_per_slab] += chunk_hist[c]
    tot = slab_tot.sum(axis=0)
    bin_start = np.concatenate([[0], np.cumsum(tot)])
    assert bin_start[-1] == n
    dest = np.empty(n, dtype=np.int64)
    for c in range(n_chunks):
        slab = c // chunks_per_slab
        before = slab_tot[:slab].sum(axis=0) + chunk_hist[slab * chunks_per_slab:c].sum(axis=0)
        gpos = bin_start[:-1] + before
        b = bins[c * clen:(c + 1) * clen]
        # stable inside the chunk: rank among the chunk's elements of the same bin
        order = np.argsort(b, kind="stable")
        rank = np.empty(b.size, dtype=np.int64)
        starts = np.concatenate([[0], np.cumsum(np.bincount(b, minlength=BINS))])[:-1]
        rank[order] = np.arange(b.size) - starts[b[order]]
        dest[c * clen:c * clen + b.size] = gpos[b] + rank
    assert np.array_equal(np.sort(dest), np.arange(n))  # every place written once
    scattered = np.empty(n, dtype=np.int64)
    scattered[dest] = np.arange(n)
    # bin sort: even bins by the bits below the common prefix of their splitters; odd bins stay
    out = scattered.copy()
    for g in range(n_split + 1):
        s, e = bin_start[2 * g], bin_start[2 * g + 1]
        if e - s < 2:
            continue
        lo, nbits = bin_bits(spl, g, keys.min(), keys.max())
        idx = scattered[s:e]
        full = keys[idx].astype(np.uint64) - np.uint64(lo)
        sub = full & np.uint64((1 << nbits) - 1 if nbits < 64 else 0xFFFFFFFFFFFFFFFF)
        assert np.array_equal(sub, full)  # (no key of the bin has a bit beyond nbits)
        out[s:e] = idx[sort_bin(sub, nbits, keys.dtype.itemsize == 8)]
    for g in range(SLOTS):  # a bin of equal keys holds equal keys
        s, e = bin_start[2 * g + 1], bin_start[2 * g + 2]
        assert e == s or np.all(keys[scattered[s:e]] == keys[scattered[s]])
    return out, bins
