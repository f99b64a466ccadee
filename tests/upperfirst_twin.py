"""CPU restatement of the rules of cunumeric_amd/csrc/upperfirst.hpp: how many upper bytes the
passes keep (upper_first_digit0), and what the fix-up does with a row that is in stable order
of its keys' upper bits (upper_first_fixup_kernel): runs of two exchanged, runs of up to 16
sorted by the whole key by the thread of their first element, an element out of order inside a
longer run calls the attempt off, runs of equal keys of any length are left alone."""
from __future__ import annotations

import numpy as np

RUN_LIMIT = 16


def digit0(kind: str, row_len: int) -> int:
    """kind: 'i' integers, 'f' float64, 'c' complex64.  Returns the first byte the passes run over."""
    spent = {"i": 0, "f": 12, "c": 15}[kind]
    need = 5 + spent
    while need < 64 and (row_len >> (need - 5 - spent)) > 1:
        need += 1
    nbytes = min(6, max(4, (need + 7) // 8))
    return 8 - nbytes


def fixup(keys: np.ndarray, pos: np.ndarray, low_bits: int):
    """keys (uint64) in stable order of keys >> low_bits, pos their payload.  Returns (keys, pos,
    done) after the fix-up's rules."""
    keys, pos = keys.copy(), pos.copy()
    n = keys.size
    up = keys >> np.uint64(low_bits)
    done = True
    # extents of the runs of equal upper bits (these never change)
    starts = np.flatnonzero(np.concatenate([[True], up[1:] != up[:-1]]))
    ends = np.concatenate([starts[1:], [n]])
    for s, e in zip(starts, ends):
        length = e - s
        if length < 2:
            continue
        seg = keys[s:e]
        if length > RUN_LIMIT:
            # nobody sorts it: any pair out of order calls the attempt off
            if np.any(seg[:-1] > seg[1:]):
                done = False
            continue
        order = np.argsort(seg, kind="stable")   # (insertion sort with strict comparisons: stable)
        keys[s:e] = seg[order]
        pos[s:e] = pos[s:e][order]
    return keys, pos, done
