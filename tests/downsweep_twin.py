"""CPU twin of one radix pass as downsweep_kernel performs it (cunumeric_amd/csrc/radix.hpp):
the same chunk / tile / wavefront geometry, the same software pipeline (tile n is ranked and
staged in step n, written out in step n+1, a last step only writes out), the same tables
(per-wave counts -> first staged slot per wave, dig_base / dig_lim / dig_oldk / old_run, the
per-digit carry of G slots) and the same per-thread slot assignment, with every array index
bounds-checked and the invariants the kernel depends on asserted:

  * a staged slot and a carry slot are never overwritten while they still hold an element
    that has not been written out,
  * the carry index of an element lies in [0, G), the elements a step writes out are
    exactly the whole 128-byte groups, every output position is written exactly once,
  * padding keys of a partial tile rank behind every real key and are never written,
  * with ``side=True`` (the digit side-band of keys-only sorts: next to every key the pass
    writes that key's digit for the NEXT pass as one byte, in whole 128-byte lines through a
    second, 128-entry carry per digit value): every byte position is written exactly once,
    a byte-carry slot lies in [0, 128) and is never overwritten while live.

It restates what the scatter pass of CUB's DeviceRadixSort does for the reference
(src/cunumeric/sort/cub_sort.cuh:60-71): a stable split of the row by one digit.
Test infrastructure only; nothing in the product imports it.
"""
from __future__ import annotations

import numpy as np

RADIX = 256


def chunk_bases(digits: np.ndarray, tile: int, tiles_per_chunk: int) -> np.ndarray:
    """What upsweep + chunk scan produce: first output position of every (chunk, digit value)."""
    n = digits.size
    clen = tile * tiles_per_chunk
    n_chunks = (n + clen - 1) // clen
    hist = np.zeros((n_chunks, RADIX), dtype=np.int64)
    for c in range(n_chunks):
        hist[c] = np.bincount(digits[c * clen:(c + 1) * clen], minlength=RADIX)
    total = hist.sum(axis=0)
    start = np.concatenate([[0], np.cumsum(total)[:-1]])
    before = np.cumsum(hist, axis=0) - hist
    return start[None, :] + before


BLINE = 128  # bytes of the side-band written at a time


def downsweep(keys: np.ndarray, pay, shift: int, nt: int, ipt: int, g: int, tiles_per_chunk: int,
              side: bool = False):
    """One pass over one row.  keys: unsigned keys; pay: payload array or None (positions are
    synthesised).  Returns (keys_out, pay_out), and with ``side`` also the side-band (the
    next pass's digit of every key written, in output order)."""
    assert nt % RADIX == 0 and (RADIX * g) % nt == 0 and g & (g - 1) == 0
    n = keys.size
    nw, tile = nt // 64, nt * ipt
    max_key = np.iinfo(keys.dtype).max
    digit_of = lambda k: (int(k) >> shift) & (RADIX - 1)
    digits = ((keys >> np.array(shift, keys.dtype)) & np.array(RADIX - 1, keys.dtype)).astype(np.int64)
    bases = chunk_bases(digits, tile, tiles_per_chunk)
    tiles_per_row = (n + tile - 1) // tile
    kout = np.zeros(n, dtype=keys.dtype)
    pout = np.zeros(n, dtype=np.int64)
    written = np.zeros(n, dtype=np.int32)
    bout = np.zeros(n, dtype=np.uint8)
    bwritten = np.zeros(n, dtype=np.int32)
    next_digit = lambda k: (int(k) >> (shift + 8)) & (RADIX - 1)

    def emit(pos, k, v):
        assert 0 <= pos < n, f"output position {pos} outside the row"
        written[pos] += 1
        kout[pos], pout[pos] = k, v

    def emit_byte(pos, b):
        assert 0 <= pos < n, f"side-band position {pos} outside the row"
        bwritten[pos] += 1
        bout[pos] = b

    for chunk in range(bases.shape[0]):
        tile0 = chunk * tiles_per_chunk
        tile_end = min(tile0 + tiles_per_chunk, tiles_per_row)
        run = bases[chunk].astype(np.int64).copy()   # owner registers (thread d < RADIX)
        carry_n = np.zeros(RADIX, dtype=np.int64)
        whist = np.zeros((nw, RADIX), dtype=np.int64)
        dig_base = np.zeros(RADIX, dtype=np.int64)
        dig_lim = np.zeros(RADIX, dtype=np.int64)
        dig_oldk = np.zeros(RADIX, dtype=np.int64)
        old_run = np.zeros(RADIX, dtype=np.int64)
        skeys = np.zeros(tile, dtype=keys.dtype)
        spay = np.zeros(tile, dtype=np.int64)
        s_live = np.zeros(tile, dtype=bool)          # checker state
        ckeys = np.zeros(RADIX * g, dtype=keys.dtype)
        cpay = np.zeros(RADIX * g, dtype=np.int64)
        c_live = np.zeros(RADIX * g, dtype=bool)     # checker state
        # side-band: owner registers and tables, byte carry
        brun = run.copy()
        b_cnt = np.zeros(RADIX, dtype=np.int64)
        b_pos = np.zeros(RADIX, dtype=np.int64)
        b_eb = np.zeros(RADIX, dtype=np.int64)
        b_delta = np.zeros(RADIX, dtype=np.int64)
        bcarry = np.zeros((RADIX, BLINE), dtype=np.uint8)
        b_live = np.zeros((RADIX, BLINE), dtype=bool)

        for tno in range(tile0, tile_end + 1):       # the step after the last tile only writes out
            has_cur = tno < tile_end
            has_prev = tno > tile0
            valid = min(tile, n - tno * tile) if has_cur else 0
            pvalid = min(tile, n - (tno - 1) * tile) if has_prev else 0
            more = tno + 1 < tile_end
            if has_prev:
                deferred = []   # byte-carry writes of carried keys: held back until the barrier
                if side:
                    # ---- side-band bytes whose 128-byte line tile n-1 completes
                    for d in range(RADIX):
                        for j in range(int(b_cnt[d])):
                            assert b_live[d, j], f"byte-carry slot {j} of digit {d} flushed but empty"
                            b_live[d, j] = False
                            emit_byte(int(b_pos[d]) + j, bcarry[d, j])
                # ---- carried elements whose group tile n-1 completes: thread x = tid + i*NT
                # holds carry slot e = x % G of digit value x // G
                for x in range(RADIX * g):
                    d, e = x // g, x % g
                    if e < dig_oldk[d]:
                        assert c_live[x], f"carry slot {e} of digit {d} flushed but empty"
                        c_live[x] = False
                        emit(int(old_run[d]) + e, ckeys[x], cpay[x])
                        if side:
                            if e < b_eb[d]:
                                emit_byte(int(old_run[d]) + e, next_digit(ckeys[x]))
                            else:
                                deferred.append((d, e - int(b_eb[d]), next_digit(ckeys[x])))
                # ---- staged tile n-1 into registers (before the barrier) ...
                staged = []
                for q in range(tile):
                    ak = skeys[q]
                    d = digit_of(ak)
                    staged.append((q, ak, spay[q], d, int(dig_base[d]), int(dig_lim[d])))
                # ---- (barrier) ... then to global memory up to the group boundary, the rest
                # to the carry
                for d, slot, b in deferred:
                    assert 0 <= slot < BLINE, f"byte-carry slot {slot} of digit {d} outside [0, {BLINE})"
                    assert not b_live[d, slot], f"byte-carry slot {slot} of digit {d} overwritten while live"
                    b_live[d, slot] = True
                    bcarry[d, slot] = b
                for q, ak, av, d, abase, alim in staged:
                    if q < pvalid:
                        assert s_live[q], f"staged slot {q} read but never written"
                        s_live[q] = False
                        if q < alim:
                            emit(abase + q, ak, av)
                            if side:
                                blim = alim - int(b_delta[d])
                                if q < blim:
                                    emit_byte(abase + q, next_digit(ak))
                                else:
                                    slot = q - blim
                                    assert 0 <= slot < BLINE, f"byte-carry slot {slot} of digit {d} outside [0, {BLINE})"
                                    assert not b_live[d, slot], f"byte-carry slot {slot} of digit {d} overwritten while live"
                                    b_live[d, slot] = True
                                    bcarry[d, slot] = next_digit(ak)
                        else:
                            e = q - alim
                            assert 0 <= e < g, f"carry index {e} of digit {d} outside [0, {g})"
                            c = d * g + e
                            assert not c_live[c], f"carry slot {e} of digit {d} overwritten while live"
                            c_live[c] = True
                            ckeys[c], cpay[c] = ak, av
                    else:
                        assert not s_live[q]
            if not has_cur:
                break
            whist[:] = 0
            off = tno * tile
            # the tile, wave-striped: thread t = wave*64 + lane, item i -> wave*64*ipt + i*64 + lane
            ck = np.full((nt, ipt), max_key, dtype=keys.dtype)
            cp = np.zeros((nt, ipt), dtype=np.int64)
            pad = np.ones((nt, ipt), dtype=bool)
            for t in range(nt):
                wave, lane = t >> 6, t & 63
                for i in range(ipt):
                    o = wave * 64 * ipt + i * 64 + lane
                    if o < valid:
                        ck[t, i], pad[t, i] = keys[off + o], False
                        cp[t, i] = (off + o) if pay is None else pay[off + o]
            # rank within the wave: wave-rows in order, lanes in order inside a row
            rank = np.zeros((nt, ipt), dtype=np.int64)
            for wave in range(nw):
                for i in range(ipt):
                    for lane in range(64):
                        t = wave * 64 + lane
                        d = digit_of(ck[t, i])
                        rank[t, i] = whist[wave, d]
                        whist[wave, d] += 1
            # ---- per-digit tile counts, first staged slot of every wave, what is written now
            count = whist.sum(axis=0)
            tile_start = np.concatenate([[0], np.cumsum(count)[:-1]])
            for d in range(RADIX):
                real = int(count[d]) - ((tile - valid) if d == RADIX - 1 else 0)
                assert real >= 0
                total = int(carry_n[d]) + real
                hi = (int(run[d]) + total) & ~(g - 1)
                flush = (hi - int(run[d]) if hi > run[d] else 0) if more else total
                assert 0 <= flush <= total
                assert more is False or (int(run[d]) + flush) % g == 0 or flush == 0
                dig_base[d] = run[d] + carry_n[d] - tile_start[d]
                dig_lim[d] = flush + tile_start[d] - carry_n[d]
                dig_oldk[d] = carry_n[d] if flush else 0
                old_run[d] = run[d]
                if side:
                    # bytes of positions [brun, run) wait in the byte carry; whole lines up
                    # to the new run position go out (everything at the end of the chunk)
                    new_run = int(run[d]) + flush
                    if more:
                        nb = new_run & ~(BLINE - 1)
                        new_brun = nb if nb > brun[d] else int(brun[d])
                    else:
                        new_brun = new_run
                    assert int(run[d]) - int(brun[d]) < BLINE
                    b_cnt[d] = int(run[d]) - int(brun[d]) if new_brun > brun[d] else 0
                    assert b_cnt[d] == 0 or new_brun >= run[d], "a flushed byte carry is flushed whole"
                    b_pos[d] = brun[d]
                    b_eb[d] = new_brun - int(run[d])
                    b_delta[d] = new_run - new_brun
                    assert 0 <= b_delta[d] < BLINE or not more
                    brun[d] = new_brun
                run[d] += flush
                carry_n[d] = total - flush
                assert 0 <= carry_n[d] < g or not more, f"carry of digit {d} does not fit {g} slots"
                off_w = int(tile_start[d])
                for w in range(nw):
                    c = int(whist[w, d])
                    whist[w, d] = off_w
                    off_w += c
            # ---- stage tile n in tile-sorted order
            for t in range(nt):
                wave = t >> 6
                for i in range(ipt):
                    d = digit_of(ck[t, i])
                    q = int(whist[wave, d] + rank[t, i])
                    assert 0 <= q < tile, f"staged slot {q} outside the tile"
                    assert not s_live[q], f"staged slot {q} overwritten while live"
                    assert pad[t, i] == (q >= valid), "padding keys take exactly the slots past valid"
                    skeys[q], spay[q] = ck[t, i], cp[t, i]
                    s_live[q] = not pad[t, i]
        assert not s_live.any() and not c_live.any(), "elements left behind at the end of the chunk"
        assert (carry_n == 0).all()
        assert not b_live.any(), "side-band bytes left behind at the end of the chunk"
        assert not side or (brun == run).all()
    assert (written == 1).all(), "an output position was not written exactly once"
    if side:
        assert (bwritten == 1).all(), "a side-band position was not written exactly once"
        return kout, pout, bout
    return kout, pout
