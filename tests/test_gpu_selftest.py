"""The hardware behaviour the radix scatter relies on without the ISA manual promising it:
the lanes of ONE returning LDS add that hit the same word are served in ascending lane
order on gfx950 (misort_selftest_lds_lane_order ranks every lane both by the returning add
and by the ballot match and counts the disagreements), and the ballot-only build of the
same sort (MISORT_RANK_BALLOT=1) gives the same results."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_lds_serves_same_word_lanes_in_lane_order():
    import torch

    from cunumeric_amd import _lib

    lib = _lib.load()
    checked, bad = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    rows = 512
    _lib.check(lib.misort_selftest_lds_lane_order(rows, ctypes.byref(checked), ctypes.byref(bad),
                                                  torch.cuda.current_stream().cuda_stream))
    assert checked.value == 6 * 512 * 16 * rows * 64   # 1.6e9 lanes
    assert bad.value == 0


def test_library_decides_the_ranking_per_gpu():
    """Before the first sort on a GPU the library probes the LDS itself; on gfx950 it finds every
    lane in order and ranks with the adds (mode 1), and the plan description says so."""
    import torch

    from cunumeric_amd import _lib

    lib = _lib.load()
    assert lib.misort_init() == 0
    mode = lib.misort_rank_mode()
    assert mode in (1, 2)
    if os.environ.get("MISORT_RANK_BALLOT", "0") in ("", "0"):
        assert mode == 1, "the probe found lanes out of order on this GPU"
    plan = _lib.describe_plan(10, 1 << 26, 1 << 26, True)
    assert ("rank=add" if mode == 1 else "rank=ballot") in plan
    assert torch.cuda.is_available()


def test_ballot_rank_gives_the_same_sort():
    """A fresh process with MISORT_RANK_BALLOT=1: the parity cases that lean on the ranking
    hardest, ranked by ballots only: every element type with three chunks per row (every
    workgroup walks several tiles), heavy ties, runs of equal keys, rows, a caller's payload,
    in place, and the headline input at 2^24."""
    code = r"""
import numpy as np, sys
sys.path.insert(0, %r)
import bench
from tests.util import ALL_DTYPES, Abi, bits_equal, random_array
abi = Abi()
abi.force_radix = True
assert abi.lib.misort_rank_mode() == 2
assert "rank=ballot" in abi.describe_plan(np.float32, 1 << 24, 1 << 24, True)
rng = np.random.default_rng(5)
for dtype in ALL_DTYPES:
    for n, chunks, narrow in ((100003, 3, False), (70001, 0, True), (300001, 5, False)):
        a = random_array(dtype, n, rng, narrow=narrow)
        print("ballot", np.dtype(dtype).name, n, chunks, narrow, flush=True)
        assert np.array_equal(abi.local_sort(a, n, argsort=True, chunks=chunks), np.argsort(a, kind="stable")), dtype
        assert bits_equal(abi.local_sort(a, n, argsort=False, chunks=chunks, inplace=True), np.sort(a, kind="stable")), dtype
for dtype in (np.int32, np.float32, np.int64):
    for copies in (16, 64, 1000):
        pool = random_array(dtype, 400000 // copies, rng, specials=False)
        a = pool[rng.integers(0, pool.size, 400000)]
        assert np.array_equal(abi.local_sort(a, a.size, argsort=True, chunks=7), np.argsort(a, kind="stable")), (dtype, copies)
a = random_array(np.float64, 5 * 120001, rng)
pay = rng.integers(-2**62, 2**62, a.size, dtype=np.int64)
perm = np.argsort(a.reshape(5, -1), axis=1, kind="stable")
got = abi.local_sort(a, 120001, argsort=True, indices_in=pay, inplace=True)
assert np.array_equal(got.reshape(5, -1), np.take_along_axis(pay.reshape(5, -1), perm, axis=1))
c2 = bench.make_c2(1 << 24, seed=2)
print("ballot C2 2^24", flush=True)
assert np.array_equal(abi.local_sort(c2, c2.size, argsort=True), np.argsort(c2, kind="stable"))
print("ballot ok")
""" % ROOT
    env = dict(os.environ, MISORT_RANK_BALLOT="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "ballot ok" in r.stdout
