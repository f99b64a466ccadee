"""Sorts of more than 2^31 elements through the C ABI: 64-bit positions in every kernel's
indexing, the 32-bit internal positions of an argsort at their limit, the counting paths
past 2^32 elements.  Inputs are generated and results checked on the device (torch), through
properties: output non-decreasing (NaN last), same multiset (histogram for 1- and 2-byte
values, sum of the bit patterns otherwise); for the argsort: a permutation whose gather is
sorted and whose ties keep their input order."""
import pytest

torch = pytest.importorskip("torch")

from cunumeric_amd import _lib  # noqa: E402

pytestmark = pytest.mark.gpu

CODES = {torch.uint8: 5, torch.int16: 2, torch.int32: 3, torch.int64: 4, torch.float32: 10}
STEP = 1 << 28


def _sorted(t):
    for s in range(0, t.numel() - 1, STEP):
        c = t[s:s + STEP + 1]
        a, b = c[:-1], c[1:]
        good = ((a <= b) | torch.isnan(b)) if t.is_floating_point() else (a <= b)
        if not bool(good.all()):
            return False
    return True


def _call(x, argsort):
    lib = _lib.load()
    dev = x.device
    n, code = x.numel(), CODES[x.dtype]
    need = lib.misort_scratch_bytes(code, n, n, int(argsort), 0)
    scratch = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    if argsort:
        out = torch.empty(n, dtype=torch.int64, device=dev)
        rc = lib.misort_local(code, x.data_ptr(), None, None, out.data_ptr(), n, n, 1, 0, scratch.data_ptr(), need, stream)
    else:
        out = torch.empty_like(x)
        rc = lib.misort_local(code, x.data_ptr(), out.data_ptr(), None, None, n, n, 1, 0, scratch.data_ptr(), need, stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    return out


def _same_histogram(x, out, k, off):
    hi = torch.zeros(k, dtype=torch.int64, device=x.device)
    ho = torch.zeros_like(hi)
    for s in range(0, x.numel(), STEP):
        hi += torch.bincount(x[s:s + STEP].to(torch.int32) + off, minlength=k)
        ho += torch.bincount(out[s:s + STEP].to(torch.int32) + off, minlength=k)
    return bool(torch.equal(hi, ho))


def test_uint8_past_2p32():
    dev = torch.device("cuda", 0)
    torch.manual_seed(1)
    n = (1 << 32) + 7
    print(f"huge uint8 sort n={n}", flush=True)
    x = torch.randint(0, 256, (n,), device=dev, dtype=torch.uint8)
    out = _call(x, False)
    assert _sorted(out) and _same_histogram(x, out, 256, 0)


def test_int16_past_2p31():
    dev = torch.device("cuda", 0)
    torch.manual_seed(2)
    n = (1 << 31) + 3
    print(f"huge int16 sort n={n}", flush=True)
    x = torch.randint(-32768, 32768, (n,), device=dev, dtype=torch.int16)
    out = _call(x, False)
    assert _sorted(out) and _same_histogram(x, out, 65536, 32768)


def test_float32_sort_and_argsort_past_2p31():
    dev = torch.device("cuda", 0)
    torch.manual_seed(3)
    n = (1 << 31) + 12345
    x = torch.randn(n, device=dev, dtype=torch.float32)
    x[::1001] = float("nan")
    x[5::997] = -0.0
    print(f"huge float32 sort n={n}", flush=True)
    out = _call(x, False)
    assert _sorted(out)
    assert int(x.view(torch.int32).sum(dtype=torch.int64)) == int(out.view(torch.int32).sum(dtype=torch.int64))
    del out
    print(f"huge float32 argsort n={n}", flush=True)
    idx = _call(x, True)
    assert int(idx.min()) == 0 and int(idx.max()) == n - 1
    seen = torch.zeros(n, dtype=torch.uint8, device=dev)
    seen[idx] = 1
    assert int(seen.sum(dtype=torch.int64)) == n, "not a permutation"
    del seen
    g = x[idx]
    assert _sorted(g)
    for s in range(0, n - 1, STEP):
        a, b = g[s:s + STEP + 1], idx[s:s + STEP + 1]
        tie = (a[:-1] == a[1:]) | (torch.isnan(a[:-1]) & torch.isnan(a[1:]))
        assert bool((~tie | (b[:-1] < b[1:])).all()), "ties not in input order"
