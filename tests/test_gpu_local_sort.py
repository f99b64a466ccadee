"""GPU parity of misort_local (through the C ABI) against the CPU oracle and NumPy.

Bit-exact: sorted values byte for byte, stable-argsort indices exactly."""
import numpy as np
import pytest

from cunumeric_amd._lib import Options
from oracle import misort_oracle as oracle
from tests.util import ALL_DTYPES, Abi, bits_equal, random_array

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=[False, True], ids=["default plan", "radix path asked for"])
def abi(request):
    # single rows of 16385 to about a million elements take the four-launch path by default;
    # the second round runs the same cases on the radix path, which serves the longer rows
    a = Abi()
    a.force_radix = request.param
    return a


SIZES_1D = [1, 2, 63, 64, 65, 255, 500, 513, 1000, 1024, 1025, 4096, 4097, 8192, 8193, 12289, 100003]


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
def test_argsort_1d_all_dtypes(abi, dtype):
    rng = np.random.default_rng(11)
    for n in SIZES_1D:
        print(f"argsort dtype={np.dtype(dtype).name} n={n}", flush=True)
        a = random_array(dtype, n, rng)
        got = abi.local_sort(a, n, argsort=True)
        assert np.array_equal(got, np.argsort(a, kind="stable")), (dtype, n)
        assert np.array_equal(got, oracle.local_sort(a, n, True)), (dtype, n)


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
def test_sort_1d_all_dtypes(abi, dtype):
    rng = np.random.default_rng(12)
    for n in SIZES_1D:
        print(f"sort dtype={np.dtype(dtype).name} n={n}", flush=True)
        a = random_array(dtype, n, rng)
        got = abi.local_sort(a, n, argsort=False)
        assert bits_equal(got, np.sort(a, kind="stable")), (dtype, n)
        got = abi.local_sort(a, n, argsort=False, inplace=True)
        assert bits_equal(got, oracle.local_sort(a, n, False)), (dtype, n)


@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.int32, np.float32, np.float64, np.int64,
                                   np.complex64], ids=lambda d: np.dtype(d).name)
def test_heavy_ties(abi, dtype):
    rng = np.random.default_rng(13)
    n = 50000
    a = random_array(dtype, n, rng, narrow=True)
    got = abi.local_sort(a, n, argsort=True)
    assert np.array_equal(got, np.argsort(a, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64], ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("copies", [16, 40, 64, 100, 256, 1000])
def test_runs_of_equal_keys_with_spread_out_digits(abi, dtype, copies):
    """Values drawn from a pool of distinct random values: every digit value is about equally
    frequent, so the scatter ranks by returning LDS adds, and the later passes meet runs of
    `copies` equal keys, where wave-rows of one or two digit values are ranked group-wise."""
    rng = np.random.default_rng(14)
    n = 1 << 20
    if np.dtype(dtype).kind == "f":
        pool = rng.standard_normal(n // copies).astype(dtype) * 1e3
    else:
        ii = np.iinfo(dtype)
        pool = rng.integers(ii.min, ii.max, n // copies, dtype=dtype)
    a = pool[rng.integers(0, pool.size, n)]
    print(f"runs dtype={np.dtype(dtype).name} copies={copies}", flush=True)
    got = abi.local_sort(a, n, argsort=True)
    assert np.array_equal(got, np.argsort(a, kind="stable"))
    assert bits_equal(abi.local_sort(a, n, argsort=False), np.sort(a, kind="stable"))
    # two rows, so that a row starts in the middle of a tile
    b = a[: 2 * 300007].reshape(2, 300007)
    got = abi.local_sort(b, 300007, argsort=True).reshape(2, -1)
    assert np.array_equal(got, np.argsort(b, axis=1, kind="stable"))


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float16, np.float32, np.int64, np.float64,
                                   np.complex128], ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("rows,row_len", [(7, 5000), (3, 12288), (64, 4096), (5, 1), (1000, 17),
                                          (300, 401), (2, 70000), (40, 700), (9, 1024), (33, 130),
                                          (70, 48)])
def test_rows(abi, dtype, rows, row_len):
    rng = np.random.default_rng(14)
    a = random_array(dtype, rows * row_len, rng)
    print(f"rows dtype={np.dtype(dtype).name} rows={rows} row_len={row_len}", flush=True)
    got = abi.local_sort(a, row_len, argsort=True, index_offset=3)
    ref = np.argsort(a.reshape(rows, row_len), axis=1, kind="stable").reshape(-1) + 3
    assert np.array_equal(got, ref)
    got = abi.local_sort(a, row_len, argsort=False)
    assert bits_equal(got, np.sort(a.reshape(rows, row_len), axis=1, kind="stable").reshape(-1))


# Radix passes cut into 3 chunks (misort_local_chunked), so that arrays of a few tiles
# already make every workgroup walk several tiles (the pipelined loop, the lines carried
# from tile to tile and the final flush) instead of the one tile per chunk that small
# arrays get by default.
FEW = 3


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=lambda d: np.dtype(d).name)
def test_multi_tile_chunks_all_dtypes(abi, dtype):
    rng = np.random.default_rng(21)
    for n in (40000, 100003, 262144):
        print(f"multi-tile dtype={np.dtype(dtype).name} n={n}", flush=True)
        a = random_array(dtype, n, rng)
        got = abi.local_sort(a, n, argsort=True, chunks=FEW)
        assert np.array_equal(got, np.argsort(a, kind="stable")), (dtype, n)
        got = abi.local_sort(a, n, argsort=False, chunks=FEW)
        assert bits_equal(got, np.sort(a, kind="stable")), (dtype, n)


@pytest.mark.parametrize("dtype", [np.uint8, np.float16, np.int32, np.float32, np.uint64, np.float64,
                                   np.complex64, np.complex128], ids=lambda d: np.dtype(d).name)
def test_multi_tile_chunks_rows_and_payload(abi, dtype):
    rng = np.random.default_rng(22)
    rows, row_len = 3, 70001
    a = random_array(dtype, rows * row_len, rng).reshape(rows, row_len)
    print(f"multi-tile rows dtype={np.dtype(dtype).name}", flush=True)
    got = abi.local_sort(a, row_len, argsort=False, chunks=FEW).reshape(rows, row_len)
    assert bits_equal(got, np.sort(a, axis=1, kind="stable"))
    got = abi.local_sort(a, row_len, argsort=True, chunks=FEW).reshape(rows, row_len)
    assert np.array_equal(got, np.argsort(a, axis=1, kind="stable"))
    # caller-provided int64 payload travels with the keys
    pay = rng.integers(-(2**62), 2**62, rows * row_len, dtype=np.int64)
    got = abi.local_sort(a, row_len, argsort=True, indices_in=pay, chunks=FEW).reshape(rows, row_len)
    ref = np.take_along_axis(pay.reshape(rows, row_len), np.argsort(a, axis=1, kind="stable"), axis=1)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", [np.uint64, np.float64, np.int32], ids=lambda d: np.dtype(d).name)
def test_default_plan_multi_tile_chunks(abi, dtype):
    """Large enough that the default plan gives every workgroup two or more tiles."""
    rng = np.random.default_rng(23)
    n = 1 << 25 if np.dtype(dtype).itemsize == 4 else 1 << 24
    a = random_array(dtype, n, rng)
    print(f"default plan multi-tile dtype={np.dtype(dtype).name} n={n}", flush=True)
    assert bits_equal(abi.local_sort(a, n, argsort=False), np.sort(a, kind="stable"))
    assert np.array_equal(abi.local_sort(a, n, argsort=True), np.argsort(a, kind="stable"))


@pytest.mark.parametrize("dtype", [np.int16, np.uint16, np.float16], ids=lambda d: np.dtype(d).name)
def test_counting_sort_of_two_byte_values(abi, dtype):
    """Long 1-D values-only sorts of 2-byte elements take the counting path: by themselves
    from 2^24 (float16) or 2^26 (integers) elements on, asked for here at a million."""
    rng = np.random.default_rng(31)
    n = (1 << 20) + 12345
    cases = {
        "random": random_array(dtype, n, rng),
        "narrow": random_array(dtype, n, rng, narrow=True),
        "constant": np.full(n, 7, dtype=dtype),
        "two far values": np.where(rng.integers(0, 2, n) == 0, 3, -3 if np.dtype(dtype).kind != "u" else 60000).astype(dtype),
        "exact multiple": random_array(dtype, 1 << 21, rng),
    }
    for name, a in cases.items():
        print(f"count16 dtype={np.dtype(dtype).name} case={name}", flush=True)
        o = Options(counting_sort=1)
        assert "strategy=count16" in abi.describe_plan(a.dtype, a.size, a.size, False, options=o)
        ref = np.sort(a, kind="stable")
        assert bits_equal(abi.local_sort(a, a.size, argsort=False, options=o), ref), name
        assert bits_equal(abi.local_sort(a, a.size, argsort=False, inplace=True, options=o), ref), name
    assert "strategy=count16" in abi.describe_plan(np.float16, 1 << 24, 1 << 24, False)
    assert "strategy=count16" not in abi.describe_plan(np.int16, 1 << 24, 1 << 24, False)
    assert "strategy=count16" in abi.describe_plan(np.int16, 1 << 26, 1 << 26, False)
    assert "strategy=count16" not in abi.describe_plan(np.int16, 1 << 26, 1 << 26, False, options=Options(counting_sort=0))


@pytest.mark.parametrize("dtype", [np.bool_, np.int8, np.uint8], ids=lambda d: np.dtype(d).name)
def test_counting_sort_of_one_byte_values(abi, dtype):
    """1-D values-only sorts of 1-byte elements beyond the row kernels take the counting path."""
    rng = np.random.default_rng(33)
    for n in (16385, 70001, (1 << 20) + 3, 1 << 22):
        for name, a in (("random", random_array(dtype, n, rng)), ("constant", np.full(n, 1, dtype=dtype))):
            print(f"count8 dtype={np.dtype(dtype).name} n={n} case={name}", flush=True)
            assert "strategy=count8" in abi.describe_plan(a.dtype, a.size, a.size, False)
            ref = np.sort(a, kind="stable")
            assert bits_equal(abi.local_sort(a, a.size, argsort=False), ref), (n, name)
            assert bits_equal(abi.local_sort(a, a.size, argsort=False, inplace=True), ref), (n, name)


def test_counting_sort_unaligned_pointers(abi):
    """Input and output that start 2 bytes past a 16-byte boundary (no 16-byte loads/stores)."""
    import torch

    rng = np.random.default_rng(32)
    n = (1 << 20) + 7
    a = random_array(np.float16, n, rng)
    dev = abi.dev
    d_in = torch.zeros(2 * (n + 8), dtype=torch.uint8, device=dev)
    d_out = torch.zeros(2 * (n + 8), dtype=torch.uint8, device=dev)
    d_in[2 : 2 + 2 * n] = torch.from_numpy(a.view(np.uint8)).to(dev)
    code = abi.to_code(a.dtype)
    need = abi.lib.misort_scratch_bytes(code, n, n, 0, 0)
    scratch = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    rc = abi.lib.misort_local(code, d_in.data_ptr() + 2, d_out.data_ptr() + 2, None, None, n, n, 1, 0,
                              scratch.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    got = d_out[2 : 2 + 2 * n].cpu().numpy().view(np.float16)
    assert bits_equal(got, np.sort(a, kind="stable"))
    assert int(d_out[:2].sum()) == 0 and int(d_out[2 + 2 * n :].sum()) == 0  # nothing written outside

    b = random_array(np.int8, n, rng)
    d_in = torch.zeros(n + 64, dtype=torch.uint8, device=dev)
    d_out = torch.zeros(n + 64, dtype=torch.uint8, device=dev)
    d_in[3 : 3 + n] = torch.from_numpy(b.view(np.uint8)).to(dev)
    code = abi.to_code(b.dtype)
    need = abi.lib.misort_scratch_bytes(code, n, n, 0, 0)
    scratch = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    rc = abi.lib.misort_local(code, d_in.data_ptr() + 3, d_out.data_ptr() + 5, None, None, n, n, 1, 0,
                              scratch.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bits_equal(d_out[5 : 5 + n].cpu().numpy().view(np.int8), np.sort(b, kind="stable"))
    assert int(d_out[:5].sum()) == 0 and int(d_out[5 + n :].sum()) == 0


def test_caller_payload(abi):
    """indices_in given: the int64 payload rides with the keys (the reference's calling
    convention, sort.cu:1744-1751), also in place."""
    rng = np.random.default_rng(15)
    for dtype in (np.int32, np.float64, np.uint8):
        n = 30000
        a = random_array(dtype, n, rng)
        payload = rng.integers(-2**62, 2**62, n, dtype=np.int64)
        order = np.argsort(a, kind="stable")
        got = abi.local_sort(a, n, argsort=True, indices_in=payload)
        assert np.array_equal(got, payload[order])
        got = abi.local_sort(a, n, argsort=True, indices_in=payload, inplace=True)
        assert np.array_equal(got, payload[order])


def test_argsort_with_values_out(abi):
    rng = np.random.default_rng(16)
    a = random_array(np.float32, 20000, rng)
    idx, vals = abi.local_sort(a, 20000, argsort=True, want_values=True)
    assert np.array_equal(idx, np.argsort(a, kind="stable"))
    assert bits_equal(vals, np.sort(a, kind="stable"))


def test_empty_and_errors(abi):
    assert abi.local_sort(np.empty(0, np.float32), 0, argsort=True).shape == (0,)
    from cunumeric_amd._lib import MisortError

    with pytest.raises(MisortError):
        abi.local_sort(np.zeros(10, np.float32), 3, argsort=False)


def test_c2_shape_medium(abi):
    """The headline input at 2^22 keys: normal floats, 1% NaN with random payloads,
    0.5% -0.0, 0.5% +0.0."""
    import bench

    a = bench.make_c2(1 << 22, seed=2)
    got = abi.local_sort(a, a.shape[0], argsort=True)
    assert np.array_equal(got, np.argsort(a, kind="stable"))


def test_golden_vectors_on_gpu(abi):
    """The committed NumPy-generated fixtures (tests/golden/) through the C ABI."""
    import os

    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sort_golden.npz"))
    for name in [k[:-3] for k in g.files if k.endswith("_in")]:
        a = g[name + "_in"]
        if name.startswith("special_"):
            dt = np.dtype(name.split("_")[1])
            a = a.view(dt) if dt.kind == "f" else a.view(f"f{dt.itemsize // 2}").view(dt).reshape(-1)
            want = g[name + "_sorted"]
            want = (want.view(dt) if dt.kind == "f"
                    else want.view(f"f{dt.itemsize // 2}").view(dt).reshape(-1))
        elif name.startswith("extremes_"):
            want = g[name + "_sorted"]
        else:
            continue
        assert np.array_equal(abi.local_sort(a, a.size, True), g[name + "_argsort"]), name
        assert bits_equal(abi.local_sort(a, a.size, False), want), name


@pytest.mark.parametrize("row_len", [17, 64, 100, 256, 400, 700, 1024, 3000, 8192])
def test_float64_rows_mostly_without_zeros_and_nans(abi, row_len):
    """Values-only float64 rows take a network on the doubles themselves unless the
    wavefront (or workgroup) holds a zero or a NaN: mix both kinds of rows."""
    rng = np.random.default_rng(77)
    rows = max(8, 60000 // row_len)
    a = rng.standard_normal((rows, row_len))
    a[rng.integers(0, rows, 3), rng.integers(0, row_len, 3)] = np.inf
    a[rng.integers(0, rows, 3), rng.integers(0, row_len, 3)] = -np.inf
    a.reshape(-1)[rng.integers(0, a.size, 40)] = 5e-324  # denormals
    a.reshape(-1)[rng.integers(0, a.size, 40)] = -5e-324
    special_rows = rng.integers(0, rows, max(1, rows // 16))
    for r in special_rows:
        a[r, rng.integers(0, row_len, 4)] = [np.nan, -0.0, 0.0, -np.nan]
    print(f"float64 rows={rows} row_len={row_len}", flush=True)
    got = abi.local_sort(a.reshape(-1), row_len, argsort=False)
    assert bits_equal(got, np.sort(a, axis=1, kind="stable").reshape(-1))


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float16, np.int32, np.float32, np.int64, np.float64,
                                   np.complex64, np.complex128], ids=lambda d: np.dtype(d).name)
def test_rows_of_random_medium_lengths(abi, dtype):
    """Rows that one workgroup sorts in its registers (1025 .. 16384 elements, less for wide keys)."""
    rng = np.random.default_rng(78)
    size = np.dtype(dtype).itemsize
    longest = 16384 if size <= 4 else (8192 if size == 8 else 4096)
    for _ in range(6):
        row_len = int(rng.integers(1025, longest + 1))
        rows = int(rng.integers(1, 4))
        print(f"medium rows dtype={np.dtype(dtype).name} rows={rows} row_len={row_len}", flush=True)
        a = random_array(dtype, rows * row_len, rng, narrow=bool(rng.integers(0, 2)))
        assert "strategy=row_block" in abi.describe_plan(a.dtype, a.size, row_len, True)
        ref = a.reshape(rows, row_len)
        got = abi.local_sort(a, row_len, argsort=True, index_offset=2)
        assert np.array_equal(got, np.argsort(ref, axis=1, kind="stable").reshape(-1) + 2)
        got = abi.local_sort(a, row_len, argsort=False, inplace=True)
        assert bits_equal(got, np.sort(ref, axis=1, kind="stable").reshape(-1))


@pytest.mark.parametrize("dtype", [np.int8, np.float16, np.int32, np.float32, np.int64, np.float64],
                         ids=lambda d: np.dtype(d).name)
def test_long_rows_that_start_off_16_byte_boundaries(abi, dtype):
    """Rows of odd length: all but the first start between 16-byte boundaries, so the
    histogram kernels take their element-by-element path there."""
    rng = np.random.default_rng(79)
    rows, row_len = 3, 70001
    a = random_array(dtype, rows * row_len, rng)
    print(f"odd rows dtype={np.dtype(dtype).name}", flush=True)
    ref = a.reshape(rows, row_len)
    got = abi.local_sort(a, row_len, argsort=True)
    assert np.array_equal(got, np.argsort(ref, axis=1, kind="stable").reshape(-1))
    got = abi.local_sort(a, row_len, argsort=False)
    assert bits_equal(got, np.sort(ref, axis=1, kind="stable").reshape(-1))
