"""misort_local_static (the entry point that allocates nothing: the scratch is a buffer the
library holds in device memory) against misort_local on the same inputs, through the C ABI,
bit for bit: two calls in a row, the second with a smaller input, so that whatever the first
call left in the shared buffer meets the second."""
import numpy as np
import pytest

from tests.util import Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20  # MISORT_STATIC_SCRATCH_BYTES in include/misort.h


def test_static_scratch_matches_caller_scratch_twice():
    abi = Abi()
    rng = np.random.default_rng(77)
    # 1. stable argsort of float32 with NaNs and signed zeros: radix passes, keys and
    #    positions ping-pong through the buffer
    n1 = 1_500_000
    a1 = random_array(np.float32, n1, rng)
    code = abi.to_code(a1.dtype)
    assert 0 < abi.lib.misort_scratch_bytes(code, n1, n1, 1, 0) <= STATIC_BYTES
    print(f"static argsort float32 n={n1}", flush=True)
    ref1 = abi.local_sort(a1, n1, argsort=True)
    got1 = abi.local_sort(a1, n1, argsort=True, static=True)
    assert np.array_equal(got1, ref1)
    assert np.array_equal(got1, np.argsort(a1, kind="stable"))
    # 2. smaller, values only: the special-value counters at the start of the buffer must be
    #    cleared by the call itself (zeros and NaNs keep their bit patterns in input order)
    n2 = 300_001
    a2 = random_array(np.float32, n2, rng)
    print(f"static sort float32 n={n2}", flush=True)
    ref2 = abi.local_sort(a2, n2, argsort=False)
    got2 = abi.local_sort(a2, n2, argsort=False, static=True)
    assert bits_equal(got2, ref2)
    assert bits_equal(got2, np.sort(a2, kind="stable"))
    # 3. rows of int64 after that, then a row-kernel shape that needs no scratch at all
    a3 = random_array(np.int64, 3 * 70_001, rng)
    print("static argsort int64 rows", flush=True)
    assert np.array_equal(abi.local_sort(a3, 70_001, argsort=True, static=True),
                          abi.local_sort(a3, 70_001, argsort=True))
    a4 = random_array(np.float64, 1000 * 256, rng)
    assert bits_equal(abi.local_sort(a4, 256, argsort=False, static=True),
                      abi.local_sort(a4, 256, argsort=False))


def test_static_scratch_refuses_what_does_not_fit():
    abi = Abi()
    t = abi.torch
    n = 1 << 24
    code = abi.to_code(np.dtype(np.float32))
    assert abi.lib.misort_scratch_bytes(code, n, n, 1, 0) > STATIC_BYTES
    d_in = t.zeros(n * 4, dtype=t.uint8, device=abi.dev)
    d_out = t.full((n * 8,), 0x5A, dtype=t.uint8, device=abi.dev)
    rc = abi.lib.misort_local_static(code, d_in.data_ptr(), None, None, d_out.data_ptr(), n, n, 1, 0,
                                     t.cuda.current_stream().cuda_stream)
    assert rc == 4  # MISORT_ERR_SCRATCH
    assert b"misort_local_static" in abi.lib.misort_last_error()
    t.cuda.synchronize()
    assert bool((d_out == 0x5A).all())  # nothing was launched
    # empty input: nothing to do
    assert abi.lib.misort_local_static(code, None, None, None, None, 0, 0, 1, 0, None) == 0


def test_static_scratch_call_allocates_nothing():
    """With inputs and outputs in place before the call, the call itself leaves the device's
    free memory and torch's own allocator untouched (the first call of the process on this GPU
    has looked the buffer's address up and probed the LDS already: misort_init)."""
    abi = Abi()
    t = abi.torch
    assert abi.lib.misort_init() == 0
    rng = np.random.default_rng(78)
    n = 400_003
    a = random_array(np.float32, n, rng)
    code = abi.to_code(a.dtype)
    d_in = t.from_numpy(a.view(np.uint8).copy()).to(abi.dev)
    d_out = t.empty(n * 8, dtype=t.uint8, device=abi.dev)
    st = t.cuda.current_stream().cuda_stream
    t.cuda.synchronize()
    free0, _ = t.cuda.mem_get_info()
    alloc0, reserved0 = t.cuda.memory_allocated(), t.cuda.memory_reserved()
    for _ in range(3):
        assert abi.lib.misort_local_static(code, d_in.data_ptr(), None, None, d_out.data_ptr(), n, n, 1, 0, st) == 0
    t.cuda.synchronize()
    free1, _ = t.cuda.mem_get_info()
    assert (t.cuda.memory_allocated(), t.cuda.memory_reserved()) == (alloc0, reserved0)
    assert free1 == free0
    assert np.array_equal(d_out.cpu().numpy().view(np.int64), np.argsort(a, kind="stable"))


def test_static_scratch_call_recorded_into_a_graph():
    """misort_init outside the capture, then misort_local_static recorded into a HIP graph
    (its launches only: the call allocates nothing, synchronises nothing and clears its
    counters with kernels, not memsets).  The graph is replayed with new inputs, eager work and
    synchronisations in between, and every replay is checked against NumPy."""
    abi = Abi()
    t = abi.torch
    assert abi.lib.misort_init() == 0
    rng = np.random.default_rng(79)
    for dtype, n, argsort in ((np.float32, 300_001, True), (np.int64, 1_200_000, False), (np.int32, 50_000, True)):
        code = abi.to_code(np.dtype(dtype))
        nbytes = n * np.dtype(dtype).itemsize
        d_in = t.zeros(nbytes, dtype=t.uint8, device=abi.dev)
        d_out = t.zeros(n * 8, dtype=t.uint8, device=abi.dev)
        a0 = random_array(dtype, n, rng)
        d_in.copy_(t.from_numpy(a0.view(np.uint8).copy()))
        # one eager call first (whatever lazy set-up the runtime does for these kernels)
        vo, io = (None, d_out.data_ptr()) if argsort else (d_out.data_ptr(), None)
        st = t.cuda.current_stream().cuda_stream
        assert abi.lib.misort_local_static(code, d_in.data_ptr(), vo, None, io, n, n, 1, 0, st) == 0
        t.cuda.synchronize()
        g = t.cuda.CUDAGraph()
        side = t.cuda.Stream()
        side.wait_stream(t.cuda.current_stream())
        with t.cuda.stream(side):
            g.capture_begin()
            rc = abi.lib.misort_local_static(code, d_in.data_ptr(), vo, None, io, n, n, 1, 0, side.cuda_stream)
            g.capture_end()
        assert rc == 0, abi.lib.misort_last_error()
        t.cuda.current_stream().wait_stream(side)
        for rep in range(4):
            a = random_array(dtype, n, rng, narrow=(rep == 2))
            d_in.copy_(t.from_numpy(a.view(np.uint8).copy()))
            d_out.zero_()
            t.cuda.synchronize()
            g.replay()
            t.cuda.synchronize()
            got = d_out.cpu().numpy()
            if argsort:
                assert np.array_equal(got.view(np.int64), np.argsort(a, kind="stable")), (dtype, rep)
            else:
                assert bits_equal(got[:nbytes].view(a.dtype), np.sort(a, kind="stable")), (dtype, rep)
            # eager work between the replays
            m = min(n, 70_001)
            assert bits_equal(abi.local_sort(a[:m], m, argsort=False), np.sort(a[:m], kind="stable"))
        del g
