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


def test_ballot_rank_gives_the_same_sort():
    """A fresh process with MISORT_RANK_BALLOT=1: the same inputs, ranked by ballots only."""
    code = r"""
import numpy as np, sys
sys.path.insert(0, %r)
from tests.util import Abi, random_array
abi = Abi()
abi.force_radix = True
assert abi.lib.misort_rank_mode() == 2
rng = np.random.default_rng(5)
for dtype, n in ((np.float32, 300001), (np.int64, 200003), (np.uint32, 1 << 20)):
    a = random_array(dtype, n, rng)
    assert np.array_equal(abi.local_sort(a, n, argsort=True), np.argsort(a, kind="stable")), dtype
    assert abi.local_sort(a, n, argsort=False).tobytes() == np.sort(a, kind="stable").tobytes(), dtype
print("ballot ok")
""" % ROOT
    env = dict(os.environ, MISORT_RANK_BALLOT="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ballot ok" in r.stdout
