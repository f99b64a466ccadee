"""The boundary is re-entrant: the reference registers its task with_concurrent(true) and runs
it on a worker thread's own stream (src/cunumeric/sort/sort.cc:73-81, sort.cu:1685).  Two host
threads sort at the same time, each on a stream of its own (neither the default one), with
scratch of its own, mixed element types and paths; every result is exact against NumPy."""
import threading

import numpy as np
import pytest

from tests.util import bits_equal, random_array

pytestmark = pytest.mark.gpu


def test_two_threads_two_streams():
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    # (dtype, elements, row length, argsort): row kernels, the four-launch path, the radix path
    # with and without positions, counting sorts, rows
    jobs = [
        (np.float32, 300_001, 300_001, True), (np.int64, 3_000_000, 3_000_000, False),
        (np.float64, 1000 * 256, 256, False), (np.uint16, 70_001, 70_001, True),
        (np.int32, 5_000_000, 5_000_000, True), (np.float16, 1 << 21, 1 << 21, False),
        (np.complex64, 200_003, 200_003, True), (np.uint8, 1 << 22, 1 << 22, False),
        (np.int32, 6 * 100_003, 100_003, True), (np.float32, 40 * 5000, 5000, False),
    ]
    errors = []
    results = {}

    def worker(wid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream(device=dev)
            rng = np.random.default_rng(900 + wid)
            order = jobs if wid == 0 else jobs[::-1]
            for rnd in range(3):
                for j, (dtype, n, row, argsort) in enumerate(order):
                    a = random_array(dtype, n, rng)
                    code = to_core_dtype(np.dtype(dtype))
                    with torch.cuda.stream(stream):
                        d_in = torch.from_numpy(a.view(np.uint8).copy()).to(dev, non_blocking=False)
                        d_v = torch.empty(a.nbytes, dtype=torch.uint8, device=dev)
                        d_i = torch.empty(n * 8, dtype=torch.uint8, device=dev)
                        need = lib.misort_scratch_bytes(code, n, row, int(argsort), 0)
                        scr = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
                        stream.synchronize()
                        rc = lib.misort_local(code, d_in.data_ptr(), None if argsort else d_v.data_ptr(), None,
                                              d_i.data_ptr() if argsort else None, n, row, 1, 0, scr.data_ptr(),
                                              need, stream.cuda_stream)
                        assert rc == 0, lib.misort_last_error()
                        stream.synchronize()
                        got = (d_i if argsort else d_v).cpu().numpy()
                    rows = a.reshape(-1, row)
                    if argsort:
                        ok = np.array_equal(got.view(np.int64).reshape(rows.shape), np.argsort(rows, axis=1, kind="stable"))
                    else:
                        ok = bits_equal(got.view(a.dtype).reshape(rows.shape), np.sort(rows, axis=1, kind="stable"))
                    if not ok:
                        errors.append(f"thread {wid} round {rnd} job {j}: {np.dtype(dtype).name} n={n} row={row} argsort={argsort}")
            results[wid] = True
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(f"thread {wid}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(w,)) for w in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=600)
    assert not errors, errors
    assert results == {0: True, 1: True}
