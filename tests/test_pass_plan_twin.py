"""CPU twin of plan_pass / input_buffer (cunumeric_amd/csrc/radix.hpp): which middle radix
passes are skipped and which of the two ping-pong buffers a pass reads, worked out by every
kernel on its own from the bits that vary over the keys.  The twin restates the rule; the
test walks a sort pass by pass for every set of dead passes and checks what the kernels rely
on: a live pass reads the buffer that the last live pass wrote and writes the other one, the
side-band a live pass writes is for the next live pass, and the flag slot it uses is not
overwritten before that pass has read it.  No GPU."""
import itertools

import pytest


def plan(varying_bytes, pass_no, n_passes):
    """(skip, parity, next_live, prev_live) as plan_pass computes them."""
    def dead(j):
        return 0 < j < n_passes - 1 and j not in varying_bytes
    parity = sum(dead(j) for j in range(1, pass_no)) & 1
    nxt = pass_no + 1
    while dead(nxt):
        nxt += 1
    prv = pass_no - 1
    while dead(prv):
        prv -= 1
    return dead(pass_no), parity, nxt, prv


def input_buffer(pass_no, parity):
    return ((pass_no - 1) & 1) ^ parity


@pytest.mark.parametrize("n_passes", [3, 4, 8, 16])
def test_every_set_of_dead_passes(n_passes):
    middle = list(range(1, n_passes - 1))
    subsets = itertools.chain.from_iterable(itertools.combinations(middle, k) for k in range(len(middle) + 1))
    if n_passes == 16:   # 2^14 subsets: a spread of them
        subsets = (s for i, s in enumerate(subsets) if i % 37 == 0)
    for dead_set in subsets:
        varying = set(range(n_passes)) - set(dead_set)
        holder = "input"          # where the data is
        side_for = None           # which pass the side-band in memory is for
        flag_owner = [None, None]  # which pass wrote each flag slot last
        last_live = None
        for k in range(n_passes):
            skip, parity, nxt, prv = plan(varying, k, n_passes)
            assert skip == (k in dead_set)
            if skip:
                continue          # moves nothing, writes no side-band and no flag
            first, last = k == 0, k == n_passes - 1
            if not first:
                assert prv == last_live
                assert holder == input_buffer(k, parity), (dead_set, k)
                # the upsweep of this pass may count the side-band: it must be the one for this pass,
                # announced in the flag slot of the pass that wrote it
                assert side_for == k and flag_owner[prv & 1] == prv, (dead_set, k)
            if last:
                holder = "output"
            else:
                out = input_buffer(k, parity) ^ 1
                assert first or out != holder
                assert not first or out == 0
                holder = out
                side_for = nxt
                flag_owner[k & 1] = k
                assert nxt > k and (nxt == n_passes - 1 or nxt not in dead_set)
            last_live = k
        assert holder == "output"
