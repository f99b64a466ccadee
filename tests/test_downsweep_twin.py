"""The CPU twin of the radix scatter kernel (tests/downsweep_twin.py) against the plain
definition of a stable split by one digit.  The twin asserts the kernel's invariants while it
runs (slot and carry indices in range, nothing overwritten while live, every output written
once); the cases cover what the kernel's index arithmetic depends on: several tiles per
chunk, a partial last tile, chunk starts that are not multiples of the carry group, digit
values that dominate, 4-, 8- and 16-byte key geometries (keys per thread and carry group as
misort.hip picks them), with and without a payload."""
import numpy as np
import pytest

from tests.downsweep_twin import RADIX, downsweep


def stable_split(keys, shift):
    d = (keys >> np.array(shift, keys.dtype)) & np.array(RADIX - 1, keys.dtype)
    order = np.argsort(d, kind="stable")
    return keys[order], order


def make(kind, n, dtype, rng):
    hi = np.iinfo(dtype).max
    if kind == "uniform":
        return rng.integers(0, hi, n, dtype=dtype, endpoint=True)
    if kind == "few":
        vals = rng.integers(0, hi, 16, dtype=dtype, endpoint=True)
        w = np.arange(1, 17, dtype=np.float64) ** -1.2
        return vals[rng.choice(16, n, p=w / w.sum())]
    if kind == "const":
        return np.full(n, rng.integers(0, hi, dtype=dtype), dtype=dtype)
    if kind == "ones":     # every key carries the digit value of the padding keys
        return np.full(n, hi, dtype=dtype)
    if kind == "runs":
        return np.sort(rng.integers(0, hi, n, dtype=dtype, endpoint=True))
    raise ValueError(kind)


# (threads, keys per thread, carry group) scaled down from the kernel's shapes
SMALL = [
    (256, 8, 32, 5 * 2048 + 77, 2),   # 4-byte keys with positions
    (256, 7, 16, 4 * 1792 + 1, 3),    # 8-byte keys with positions: odd keys per thread
    (256, 16, 32, 3 * 4096, 2),       # 4-byte keys only, whole tiles
    (256, 4, 8, 300, 4),              # 16-byte keys; a single partial tile
    (512, 3, 16, 7 * 1536 + 5, 7),    # one chunk walks every tile
]


@pytest.mark.parametrize("kind", ["uniform", "few", "const", "ones", "runs"])
@pytest.mark.parametrize("nt,ipt,g,n,tpc", SMALL)
def test_twin_matches_stable_split(kind, nt, ipt, g, n, tpc):
    dtype = np.uint64 if g <= 16 else np.uint32
    rng = np.random.default_rng(hash((kind, nt, ipt, n)) & 0xFFFF)
    keys = make(kind, n, dtype, rng)
    for shift in (0, 8 * (np.dtype(dtype).itemsize - 1)):
        got_k, got_p = downsweep(keys, None, shift, nt, ipt, g, tpc)
        ref_k, ref_p = stable_split(keys, shift)
        assert np.array_equal(got_k, ref_k)
        assert np.array_equal(got_p, ref_p)


@pytest.mark.parametrize("nt,ipt,g,dtype", [(1024, 8, 32, np.uint32), (1024, 7, 16, np.uint64)],
                         ids=["u32+idx32", "u64+idx32"])
def test_twin_kernel_geometry_with_payload(nt, ipt, g, dtype):
    """The kernel's own shapes over two chunks with a partial last tile, carrying a payload
    from an earlier pass."""
    rng = np.random.default_rng(5)
    n = 3 * nt * ipt + 1234
    keys = rng.integers(0, np.iinfo(dtype).max, n, dtype=dtype)
    pay = rng.permutation(n).astype(np.int64)
    got_k, got_p = downsweep(keys, pay, 8, nt, ipt, g, 2)
    ref_k, order = stable_split(keys, 8)
    assert np.array_equal(got_k, ref_k)
    assert np.array_equal(got_p, pay[order])


@pytest.mark.parametrize("kind", ["uniform", "few", "const", "ones", "runs"])
@pytest.mark.parametrize("nt,ipt,g,n,tpc", [
    (256, 16, 32, 5 * 4096 + 77, 2),   # 4-byte keys only
    (256, 7, 16, 9 * 1792 + 1, 4),     # 8-byte keys only, odd keys per thread
    (256, 8, 16, 6 * 2048 + 9, 3),     # 8-byte keys only, the kernel's keys per thread
    (256, 7, 16, 300, 4),              # a single partial tile
    (512, 3, 16, 40 * 1536 + 5, 40),   # one chunk walks many tiles: lines complete every few steps
    (256, 2, 16, 64 * 512 + 3, 16),    # two keys of a digit value per tile: the byte carry fills slowly
])
def test_twin_digit_side_band(kind, nt, ipt, g, n, tpc):
    """Keys-only passes also write every key's digit for the next pass as a byte, in output
    order, through the 128-entry byte carry: the bytes must be the next digit of the keys
    where the pass put them, every position written once (asserted inside the twin)."""
    dtype = np.uint64 if g <= 16 else np.uint32
    rng = np.random.default_rng(hash((kind, nt, ipt, n, "side")) & 0xFFFF)
    keys = make(kind, n, dtype, rng)
    for shift in (0, 8 * (np.dtype(dtype).itemsize - 2)):
        got_k, got_p, got_b = downsweep(keys, None, shift, nt, ipt, g, tpc, side=True)
        ref_k, ref_p = stable_split(keys, shift)
        assert np.array_equal(got_k, ref_k)
        assert np.array_equal(got_p, ref_p)
        nxt = (ref_k >> np.array(shift + 8, dtype)) & np.array(RADIX - 1, dtype)
        assert np.array_equal(got_b, nxt.astype(np.uint8))
