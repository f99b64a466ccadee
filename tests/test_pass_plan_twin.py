"""CPU twin of plan_pass / input_buffer (cunumeric_amd/csrc/radix.hpp): which radix
passes are skipped and which of the two ping-pong buffers a pass reads, worked out by every
kernel on its own from the bits that vary over the keys.  The twin restates the rule; the
test walks a sort pass by pass for every set of dead passes and checks what the kernels rely
on: a live pass reads the buffer that the last live pass wrote and writes the other one, the
side-band a live pass writes is for the next live pass, and the flag slot it uses is not
overwritten before that pass has read it.  No GPU."""
import itertools

import pytest


def plan(varying_bytes, pass_no, n_passes, early_last=0, base=0):
    """(skip, parity, next_live, prev_live, is_last) as plan_pass computes them; early_last: the
    highest pass that may write the result in place of the top pass (0: none); base: pass j runs
    over byte base + j of the key (PassParams::digit_base: sorts by the upper bytes only)."""
    last = n_passes - 1
    if early_last:
        while last > 0 and last + base not in varying_bytes:
            last -= 1
        if last == 0 or last > early_last:
            last = n_passes - 1
    def dead(j):
        return j > last or (0 < j < last and j + base not in varying_bytes)
    parity = sum(dead(j) for j in range(1, pass_no)) & 1
    nxt = pass_no + 1
    while nxt < last and dead(nxt):
        nxt += 1
    prv = pass_no - 1
    while prv > 0 and dead(prv):
        prv -= 1
    return dead(pass_no), parity, nxt, prv, pass_no == last


def input_buffer(pass_no, parity):
    return ((pass_no - 1) & 1) ^ parity


@pytest.mark.parametrize("early", [False, True])
@pytest.mark.parametrize("n_passes", [3, 4, 8, 16])
def test_every_set_of_dead_passes(n_passes, early):
    """Bytes 1 .. n-1 constant in every combination (byte 0 is never looked at: pass 0 always
    runs).  Without early_last the top pass runs whatever its byte does."""
    others = list(range(1, n_passes))
    subsets = itertools.chain.from_iterable(itertools.combinations(others, k) for k in range(len(others) + 1))
    if n_passes == 16:   # 2^15 subsets: a spread of them
        subsets = (s for i, s in enumerate(subsets) if i % 37 == 0)
    for constant in subsets:
        varying = set(range(n_passes)) - set(constant)
        early_last = n_passes // 2 if early else 0   # what the host passes
        live_after_0 = [j for j in range(1, n_passes) if j in varying]
        if early_last and live_after_0 and live_after_0[-1] <= early_last:
            writer = live_after_0[-1]
        else:
            writer = n_passes - 1
        runs = {0, writer} | {j for j in live_after_0 if j < writer}
        holder = "input"          # where the data is
        side_for = None           # which pass the side-band in memory is for
        flag_owner = [None, None]  # which pass wrote each flag slot last
        last_live = None
        for k in range(n_passes):
            skip, parity, nxt, prv, is_last = plan(varying, k, n_passes, early_last)
            assert skip == (k not in runs), (constant, k)
            assert is_last == (k == writer)
            if skip:
                continue          # moves nothing, writes no side-band and no flag
            first = k == 0
            if not first:
                assert prv == last_live
                assert holder == input_buffer(k, parity), (constant, k)
                # the upsweep of this pass may count the side-band: it must be the one for this pass,
                # announced in the flag slot of the pass that wrote it
                assert side_for == k and flag_owner[prv & 1] == prv, (constant, k)
            if is_last:
                holder = "output"
            else:
                out = input_buffer(k, parity) ^ 1
                assert first or out != holder
                assert not first or out == 0
                holder = out
                side_for = nxt
                flag_owner[k & 1] = k
                assert nxt > k and nxt in runs
            last_live = k
        assert holder == "output"


@pytest.mark.parametrize("base", [2, 3, 4])
def test_sorts_by_the_upper_bytes_only(base):
    """Passes over bytes base .. 7 of an 8-byte key (the attempt of upperfirst.hpp): what varies
    in the bytes below base plays no part, pass 0 (byte `base`) always runs, the pass over byte 7
    writes the result, and the buffers alternate over the live passes as in a sort of all bytes."""
    n_passes = 8 - base
    upper = list(range(base + 1, 8))
    for k in range(len(upper) + 1):
        for constant in itertools.combinations(upper, k):
            for low in (set(), set(range(base))):   # the lower bytes constant, or all varying
                varying = (set(range(base, 8)) - set(constant)) | low
                runs = {0, n_passes - 1} | {j for j in range(1, n_passes - 1) if j + base in varying}
                holder, last_live = "input", None
                for j in range(n_passes):
                    skip, parity, nxt, prv, is_last = plan(varying, j, n_passes, 0, base)
                    assert skip == (j not in runs), (base, constant, j)
                    assert is_last == (j == n_passes - 1)
                    if skip:
                        continue
                    if j:
                        assert prv == last_live and holder == input_buffer(j, parity)
                    if is_last:
                        holder = "output"
                    else:
                        holder = input_buffer(j, parity) ^ 1 if j else 0
                        assert nxt in runs and nxt > j   # the side-band is for byte base + nxt
                    last_live = j
                assert holder == "output"
