#!/usr/bin/env python3
"""Headline benchmark: stable argsort of 2^28 float32 keys on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--log2n 28]

One "step" is one call of the hot path (misort_local through the C ABI) over the whole
batch: float32 keys in HBM -> int64 stable-argsort indices in HBM.  Prints ONE JSON line.
--workload selects one of the other benchmark inputs (c1, c3, c3t, c4, c5a, c5b, i64, f64) for the
same line format; the default, c2, is the headline.  Every run of these workloads ends with
plain 1 GiB device copies: their rate is reported beside the roofline, and they give
hardware-counter runs a kernel of known traffic to scale by (--calib-copy is accepted for
older command lines and changes nothing).

Workload (the headline configuration): N = 2^28 float32, 98 % standard normal, 1 % NaN
with random sign and payload bits, 0.5 % -0.0 and 0.5 % +0.0 at random positions, from a
seeded PCG64.  Inputs are resident in HBM and outputs / scratch pre-allocated before the
timed region.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
METRIC = "Gkeys/s + % of HBM peak, stable argsort fp32 N=2^28, 1 MI355X"


# ---------------------------------------------------------------------------------------
# synthetic workloads (shared with the tests)
# ---------------------------------------------------------------------------------------
def make_c1(n: int = 1 << 24, seed: int = 1) -> np.ndarray:
    """1-D int32 over the full range."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(-(2**31), 2**31, n, dtype=np.int32)


def make_c2(n: int = 1 << 28, seed: int = 2) -> np.ndarray:
    """float32: 98 % N(0,1), 1 % NaN (random sign / payload), 0.5 % -0.0, 0.5 % +0.0,
    positions interleaved by a random permutation."""
    rng = np.random.Generator(np.random.PCG64(seed))
    x = rng.standard_normal(n, dtype=np.float32)
    p = rng.permutation(n)
    n_nan, n_z = n // 100, n // 200
    bits = x.view(np.uint32)
    sign = rng.integers(0, 2, n_nan, dtype=np.uint32) << np.uint32(31)
    mant = rng.integers(1, 2**23, n_nan, dtype=np.uint32)
    bits[p[:n_nan]] = sign | np.uint32(0x7F800000) | mant
    bits[p[n_nan : n_nan + n_z]] = np.uint32(0x80000000)
    bits[p[n_nan + n_z : n_nan + 2 * n_z]] = np.uint32(0)
    return x


def make_c3(rows: int = 1 << 20, cols: int = 256, seed: int = 3) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.random((rows, cols))


def make_c4(n: int = 1 << 28, seed: int = 4) -> np.ndarray:
    """int64 Zipf(s=1.2) over 16 distinct values scattered across the int64 range."""
    rng = np.random.Generator(np.random.PCG64(seed))
    v = rng.integers(-(2**63), 2**63, 16, dtype=np.int64)
    w = np.arange(1, 17, dtype=np.float64) ** -1.2
    return v[rng.choice(16, n, p=w / w.sum())]


def make_uniform_int64(n: int = 1 << 28, seed: int = 9) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(-(2**63), 2**63 - 1, n, dtype=np.int64, endpoint=True)


def make_normal_float64(n: int = 1 << 28, seed: int = 10) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal(n)


def make_small_int64(n: int = 1 << 28, seed: int = 8) -> np.ndarray:
    """int64 values from a small range (labels, indices, counts: what NumPy's default integer
    usually holds): the upper six key bytes are the same in every element."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(0, 50000, n, dtype=np.int64)


def make_c5a(n: int = 1 << 26, seed: int = 5) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    pool = np.unique(rng.standard_normal(4096, dtype=np.float32))[:1024]
    out = np.empty(n, dtype=np.complex64)
    out.real = pool[rng.integers(0, 1024, n)]
    out.imag = rng.standard_normal(n, dtype=np.float32)
    return out


def make_c5b(n: int = 1 << 30, seed: int = 6) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    out = np.empty(n, dtype=np.float16)
    step = 1 << 26
    for s in range(0, n, step):
        e = min(n, s + step)
        out[s:e] = (rng.random(e - s, dtype=np.float32) * 2 - 1).astype(np.float16)
    return out


# ---------------------------------------------------------------------------------------
# CPU baseline: the reference's CPU/OpenMP variant restated over Thrust's host back-ends
# ---------------------------------------------------------------------------------------
def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def cpu_physical_cores() -> int:
    """Distinct (package, core) pairs among the CPUs this process may run on."""
    try:
        allowed = os.sched_getaffinity(0)
        cores, cur = set(), {}
        with open("/proc/cpuinfo") as f:
            for line in f.read().split("\n") + [""]:
                if ":" in line:
                    k, v = [x.strip() for x in line.split(":", 1)]
                    cur[k] = v
                elif cur:
                    if int(cur.get("processor", -1)) in allowed:
                        cores.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
                    cur = {}
        return len(cores) or len(allowed)
    except (OSError, ValueError, AttributeError):
        return os.cpu_count() or 1


def cpu_baseline(sample: np.ndarray, code: int, row: int, argsort: bool, threads: int) -> dict:
    """The reference's CPU/OpenMP variant (oracle/cpu_variant.cc: Thrust stable sort per row
    under omp::par, as in sort_cpu.inl:40-69) timed on `threads` host cores: median of three
    runs of std::chrono-equivalent wall time around the sort call only."""
    path = os.path.join(ROOT, "oracle", "libcpu_variant.so")
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    host = (f"{cpu_model()}; {os.cpu_count()} logical CPUs on the host, {usable} usable by this process on "
            f"{cpu_physical_cores()} physical cores; {threads} OpenMP threads used")
    if not os.path.exists(path):
        return {"value": None, "unit": "Gkeys/s", "cores": threads, "kind": "port", "host": host,
                "sample": "oracle/libcpu_variant.so not built"}
    lib = ctypes.CDLL(path)
    lib.cpu_variant_sort.restype = ctypes.c_int
    lib.cpu_variant_sort.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t,
                                     ctypes.c_int, ctypes.c_int]
    n = sample.size
    note = ""
    if sample.dtype.kind in "fc":
        # Thrust's OpenMP merge sort compares with operator<, under which NaNs are unordered:
        # its result on them is not a sort (and not what NumPy returns).  The baseline sorts the
        # same input with every NaN replaced by a finite value, so that it times a real sort.
        nan = np.isnan(sample)
        if nan.any():
            sample = sample.copy()
            sample[nan] = 0.5
            note = f"; its {int(nan.sum())} NaNs replaced by 0.5 (Thrust's omp merge sort does not order NaNs)"
    vals = np.empty_like(sample)
    idx = np.empty(n, dtype=np.int64) if argsort else None
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        rc = lib.cpu_variant_sort(code, sample.ctypes.data, vals.ctypes.data,
                                  idx.ctypes.data if argsort else None, n, row, 1,
                                  1 if threads > 1 else 0)
        dt = time.perf_counter() - t0
        if rc != 0:
            return {"value": None, "unit": "Gkeys/s", "cores": threads, "kind": "port", "host": host,
                    "sample": "dtype not covered by the CPU variant port"}
        times.append(dt)
    med = float(np.median(times))
    return {
        "value": n / med / 1e9,
        "unit": "Gkeys/s",
        "cores": threads,
        "kind": "port",
        "host": host,
        "sample": f"first {n} elements of the same input (rows of {row}){note}; thrust::stable_sort"
                  f"{'_by_key (int64 payload)' if argsort else ''} per row, omp::par, as in "
                  f"sort_cpu.inl:40-69; median of 3 runs: {med*1e3:.0f} ms "
                  f"({', '.join(f'{t*1e3:.0f}' for t in times)})",
    }


# ---------------------------------------------------------------------------------------
# workloads: generator, default log2 of the element count, argsort?, row length (0 = 1-D)
# ---------------------------------------------------------------------------------------
WORKLOADS = {
    "c1": ("C1: 1-D int32 full range, sort (keys only)", make_c1, 24, False, 0),
    "c2": ("C2: 1-D float32 stable argsort, 98% N(0,1) + 1% NaN (random payload) + 0.5% -0.0 "
           "+ 0.5% +0.0, int64 indices", make_c2, 28, True, 0),
    "c3": ("C3: float64 (rows, 256), sort along the last axis", None, 28, False, 256),
    "c3t": ("C3: float64 (2^20, 256), sort along axis 0 through the host API (transposed "
            "copy, row sort, transposed copy back)", None, 28, False, -1),
    "c4": ("C4: 1-D int64, 16 distinct values (Zipf 1.2), stable argsort", make_c4, 28, True, 0),
    "c5a": ("C5a: 1-D complex64, 1024 distinct real parts, stable argsort", make_c5a, 26, True, 0),
    "c5b": ("C5b: 1-D float16 uniform(-1,1), sort (keys only)", make_c5b, 30, False, 0),
    "i64small": ("1-D int64 below 50000, stable argsort (six of the eight radix passes see one "
                 "digit value and are skipped)", make_small_int64, 28, True, 0),
    "i64": ("1-D int64 full range, stable argsort (the radix passes run over the upper five key "
            "bytes, one read of the result sorts the runs of equal upper bytes)", make_uniform_int64, 28, True, 0),
    "f64": ("1-D float64 N(0,1), stable argsort (radix passes over the upper six key bytes first)",
            make_normal_float64, 28, True, 0),
}

# HBM bytes per launch of the downsweep kernel on the headline workload (N = 2^28), from
# the FETCH_SIZE / WRITE_SIZE hardware counters scaled by what the same counters read for
# a 1 GiB copy; profiles/downsweep_c2_f32_argsort_2p28_hbm_traffic.md holds the runs.
C2_DOWNSWEEP_TRAFFIC_BYTES_PER_LAUNCH = 4.153e9  # 1.752 GiB read + 2.116 GiB written


def algorithmic_bytes_per_key(k: int, v: int, role: str) -> int:
    """Bytes an LSD radix pass has to move per key (k key bytes, v index bytes)."""
    if v == 0:
        return 2 * k
    return {"downsweep_first": 2 * k + v, "downsweep_middle": 2 * k + 2 * v,
            "downsweep_last": k + 2 * v, "downsweep_only": k + v}[role]


def run_searchsorted(args) -> int:
    """--workload ss: 2^24 float32 queries into a sorted array of 2^log2n float32
    (searchsorted is the step after the sort path; not the headline)."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    log2n = args.log2n if args.log2n is not None else 28
    n, m = 1 << log2n, 1 << 24
    rng = np.random.Generator(np.random.PCG64(7))
    a = np.sort(rng.standard_normal(n, dtype=np.float32))
    v = rng.standard_normal(m, dtype=np.float32)
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_v = torch.from_numpy(v.view(np.uint8)).to(dev)
    d_o = torch.empty(m * 8, dtype=torch.uint8, device=dev)
    code = to_core_dtype(np.float32)
    stream = torch.cuda.current_stream().cuda_stream

    need = lib.misort_searchsorted_scratch_bytes(code, n, m)  # > 0: the queries are sorted first
    d_s = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)

    def plain():
        _lib.check(lib.misort_searchsorted(code, d_a.data_ptr(), n, d_v.data_ptr(), m, 1,
                                           d_o.data_ptr(), stream))

    def step():
        _lib.check(lib.misort_searchsorted_ws(code, d_a.data_ptr(), n, d_v.data_ptr(), m, 1,
                                              d_o.data_ptr(), d_s.data_ptr() if need else None, need, stream))

    def timed(f):
        for _ in range(args.warmup):
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            f()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    dt_plain = timed(plain)
    ref = np.searchsorted(a, v[: 1 << 20], side="left")
    ok = bool(np.array_equal(d_o.cpu().numpy().view(np.int64)[: 1 << 20], ref))
    d_o.zero_()
    dt = timed(step)
    got = d_o.cpu().numpy().view(np.int64)
    ok = ok and bool(np.array_equal(got[: 1 << 20], ref))
    probes = max(log2n - 14, 0)  # global probes per query after the 16384-entry LDS table
    t1 = time.perf_counter()
    np.searchsorted(a, v[: 1 << 22], side="left")
    cpu = (1 << 22) / (time.perf_counter() - t1) / 1e9
    out = {
        "metric": f"Gqueries/s, searchsorted of 2^24 float32 into 2^{log2n} sorted float32, 1 MI355X",
        "value": m / dt / 1e9, "unit": "Gqueries/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": f"searchsorted, side=left, n=2^{log2n}, m=2^24, random queries",
                   "queries_sorted_first": bool(need)},
        "ms_per_step_without_workspace": dt_plain * 1e3,
        "parity_guard": "ok" if ok else "FAILED",
        # latency-bound: each query makes `probes` dependent 4-byte reads at random places;
        # priced as one 64-byte memory sector per probe plus the query and the answer
        "roofline": {"bound": "hbm", "kernel": "searchsorted", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "achieved": m * (probes * 64 + 12) / dt / 1e9,
                     "frac": m * (probes * 64 + 12) / dt / 1e9 / HBM_PEAK_GBS, "traffic": None},
        "cpu_baseline": {"value": cpu, "unit": "Gqueries/s", "cores": 1, "kind": "port",
                         "sample": "numpy.searchsorted, first 2^22 queries, same sorted array"},
    }
    print(json.dumps(out))
    return 0 if ok else 1


def run_unique(args) -> int:
    """--workload uniq: unique of 2^log2n int32 drawn from 2^20 distinct values
    (unique is a consumer of the values-only sort; not the headline)."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    log2n = args.log2n if args.log2n is not None else 28
    n = 1 << log2n
    rng = np.random.Generator(np.random.PCG64(8))
    pool = rng.integers(-(2**31), 2**31, 1 << 20, dtype=np.int32)
    a = pool[rng.integers(0, 1 << 20, n)]
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_o = torch.empty(n * 4, dtype=torch.uint8, device=dev)
    d_c = torch.zeros(1, dtype=torch.int64, device=dev)
    code = to_core_dtype(np.int32)
    need = lib.misort_unique_scratch_bytes(code, n)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        _lib.check(lib.misort_unique(code, d_a.data_ptr(), d_o.data_ptr(), d_c.data_ptr(), n,
                                     scratch.data_ptr(), need, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    k = int(d_c.item())
    got = d_o[: 4 * k].cpu().numpy().view(np.int32)
    # guard: strictly increasing, every element one of the pool's values, and every value
    # of a leading sample of the input present (the exact comparison lives in tests/)
    ok = bool(np.all(got[:-1] < got[1:])) and bool(np.isin(got, pool).all())
    ok = ok and bool(np.isin(np.unique(a[: 1 << 22]), got).all())
    sample = a[: 1 << 25]
    t1 = time.perf_counter()
    np.unique(sample)
    cpu = sample.size / (time.perf_counter() - t1) / 1e9
    b = 4 + 2 * 4 * 4 + 4  # one histogram read, four passes, the compaction's read
    out = {
        "metric": f"Gkeys/s, unique of 2^{log2n} int32 (2^20 distinct values), 1 MI355X",
        "value": n / dt / 1e9, "unit": "Gkeys/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": f"unique, int32, n=2^{log2n}, {k} distinct values found"},
        "parity_guard": "ok" if ok else "FAILED",
        "roofline": {"bound": "hbm", "kernel": "downsweep_kernel", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "achieved": b * n / dt / 1e9, "frac": b * n / dt / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "note": "whole call: values-only radix sort (36 B/key) + one compaction read"},
        "cpu_baseline": {"value": cpu, "unit": "Gkeys/s", "cores": 1, "kind": "port",
                         "sample": "numpy.unique of the first 2^25 elements"},
    }
    print(json.dumps(out))
    return 0 if ok else 1


def run_partition(args) -> int:
    """--workload part: argpartition of 2^log2n float32 (the C2 input) around the median
    (selection instead of the reference's full sort; not the headline)."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    log2n = args.log2n if args.log2n is not None else 28
    n = 1 << log2n
    kth = n // 2
    a = make_c2(n, seed=2)
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_o = torch.empty(n * 8, dtype=torch.uint8, device=dev)
    code = to_core_dtype(np.float32)
    need = lib.misort_partition_scratch_bytes(code, n, n, 1, kth)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        _lib.check(lib.misort_partition(code, d_a.data_ptr(), None, d_o.data_ptr(), n, n, kth, 0,
                                        scratch.data_ptr(), need, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    idx = d_o.cpu().numpy().view(np.int64)
    from oracle import misort_oracle as oracle  # checker only

    keys = oracle.to_key(a)[0]
    got = keys[idx]
    pivot = np.partition(keys, kth)[kth]
    ok = bool(got[kth] == pivot) and bool(np.all(got[:kth] <= pivot)) and bool(np.all(got[kth:] >= pivot))
    ok = ok and bool(np.array_equal(np.sort(idx), np.arange(n)))
    sample = a[: 1 << 25]
    t1 = time.perf_counter()
    np.argpartition(sample, sample.size // 2)
    cpu = sample.size / (time.perf_counter() - t1) / 1e9
    # two select passes over the row (the other two read the few keys that still match), the
    # split's read and its int64 write
    b = 2 * 4 + (4 + 8)
    out = {
        "metric": f"Gkeys/s, argpartition (median) of 2^{log2n} float32, 1 MI355X",
        "value": n / dt / 1e9, "unit": "Gkeys/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": f"argpartition, float32 (C2 input), n=2^{log2n}, kth=n/2, int64 positions"},
        "parity_guard": "ok" if ok else "FAILED",
        "roofline": {"bound": "hbm", "kernel": "select_hist + select_split", "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "achieved": b * n / dt / 1e9, "frac": b * n / dt / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "note": "whole call, 20 algorithmic bytes per key"},
        "cpu_baseline": {"value": cpu, "unit": "Gkeys/s", "cores": 1, "kind": "port",
                         "sample": "numpy.argpartition of the first 2^25 elements"},
    }
    print(json.dumps(out))
    return 0 if ok else 1


def run_select(args) -> int:
    """--workload sel: the two middle order statistics and the largest element of 2^log2n
    float32 (the C2 input) by selection, which is what quantile / percentile / median need of
    the sort (the reference sorts the array for them; not the headline)."""
    import torch

    import cunumeric_amd as num
    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    log2n = args.log2n if args.log2n is not None else 28
    n = 1 << log2n
    kth = n // 2 - 1
    a = make_c2(n, seed=2)
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_o = torch.zeros(3 * 4, dtype=torch.uint8, device=dev)
    code = to_core_dtype(np.float32)
    need = lib.misort_select_scratch_bytes(code, n, n, kth)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        _lib.check(lib.misort_select(code, d_a.data_ptr(), n, n, kth, d_o.data_ptr(), d_o.data_ptr() + 4,
                                     d_o.data_ptr() + 8, scratch.data_ptr(), need, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    got = d_o.cpu().numpy().view(np.float32)
    sample = a[: 1 << 25]
    t1 = time.perf_counter()
    np.partition(sample, [sample.size // 2 - 1, sample.size // 2])
    cpu = sample.size / (time.perf_counter() - t1) / 1e9
    ref = np.partition(a, [kth, kth + 1])  # NaNs order last in NumPy too
    ok = bool(got[0] == ref[kth]) and bool(got[1] == ref[kth + 1]) and bool(np.isnan(got[2]))
    # the Python caller, end to end (allocations, the blend and the NaN test through torch)
    d_arr = num.array(a)
    med = float(np.asarray(num.quantile(d_arr, 0.5)))
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for _ in range(args.steps):
        num.quantile(d_arr, 0.5)
    torch.cuda.synchronize()
    dq = (time.perf_counter() - t2) / args.steps
    ok = ok and np.isnan(med)  # the input holds NaNs: no quantile, as in NumPy
    b = 2 * 4  # two selection passes over the row (the rest reads the few keys that still match)
    out = {
        "metric": f"Gkeys/s, elements kth, kth+1 and last in sort order of 2^{log2n} float32, 1 MI355X",
        "value": n / dt / 1e9, "unit": "Gkeys/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": f"select, float32 (C2 input), n=2^{log2n}, kth=n/2-1"},
        "parity_guard": "ok" if ok else "FAILED",
        "quantile_call_ms": dq * 1e3,
        "roofline": {"bound": "hbm", "kernel": "select_hist", "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "achieved": b * n / dt / 1e9, "frac": b * n / dt / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "note": "whole call, 8 algorithmic bytes per key"},
        "cpu_baseline": {"value": cpu, "unit": "Gkeys/s", "cores": 1, "kind": "port",
                         "sample": "numpy.partition around the two middle positions of the first 2^25 elements"},
    }
    print(json.dumps(out))
    return 0 if ok else 1


def run_axis(args) -> int:
    """--workload axis: sort of a float32 (k, 2^log2n / k) array along axis 0, k = 256: the
    column kernel, with the transposed route (swap, row sort, swap: what the reference does)
    timed beside it (not the headline)."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    log2n = args.log2n if args.log2n is not None else 28
    n, k = 1 << log2n, 256
    inner = n // k
    a = make_c2(n, seed=5)
    d_a = torch.from_numpy(a.view(np.uint8)).to(dev)
    d_o = torch.empty(n * 4, dtype=torch.uint8, device=dev)
    d_t = torch.empty(n * 4, dtype=torch.uint8, device=dev)
    code = to_core_dtype(np.float32)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.misort_scratch_bytes(code, n, k, 0, 0)
    scratch = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)

    def step():
        _lib.check(lib.misort_sort_axis(code, d_a.data_ptr(), d_o.data_ptr(), None, 1, k, inner, 0, stream))

    def step_swapped():
        _lib.check(lib.misort_swap_last(d_a.data_ptr(), d_t.data_ptr(), 1, k, 1, inner, 4, stream))
        _lib.check(lib.misort_local(code, d_t.data_ptr(), d_t.data_ptr(), None, None, n, k, 1, 0,
                                    scratch.data_ptr(), need, stream))
        _lib.check(lib.misort_swap_last(d_t.data_ptr(), d_o.data_ptr(), 1, inner, 1, k, 4, stream))

    def timed(f):
        for _ in range(args.warmup):
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            f()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    d_i = torch.empty(n * 8, dtype=torch.uint8, device=dev)
    d_it = torch.empty(n * 8, dtype=torch.uint8, device=dev)
    need_arg = lib.misort_scratch_bytes(code, n, k, 1, 0)
    scratch_arg = torch.empty(max(need_arg, 256), dtype=torch.uint8, device=dev)

    def step_arg():
        _lib.check(lib.misort_sort_axis(code, d_a.data_ptr(), None, d_i.data_ptr(), 1, k, inner, 0, stream))

    def step_arg_swapped():
        _lib.check(lib.misort_swap_last(d_a.data_ptr(), d_t.data_ptr(), 1, k, 1, inner, 4, stream))
        _lib.check(lib.misort_local(code, d_t.data_ptr(), None, None, d_it.data_ptr(), n, k, 1, 0,
                                    scratch_arg.data_ptr(), need_arg, stream))
        _lib.check(lib.misort_swap_last(d_it.data_ptr(), d_i.data_ptr(), 1, inner, 1, k, 8, stream))

    dt_arg_swapped = timed(step_arg_swapped)
    arg_swapped = d_i.cpu().numpy().copy()
    dt_arg = timed(step_arg)
    arg_ok = d_i.cpu().numpy().tobytes() == arg_swapped.tobytes()
    del arg_swapped
    dt_swapped = timed(step_swapped)
    swapped = d_o.cpu().numpy().view(np.float32).copy()
    dt = timed(step)
    got = d_o.cpu().numpy().view(np.float32)
    cols = min(inner, 1 << 14)
    sample = np.ascontiguousarray(a.reshape(k, inner)[:, :cols])
    t1 = time.perf_counter()
    ref = np.sort(sample, axis=0, kind="stable")
    cpu = sample.size / (time.perf_counter() - t1) / 1e9
    ok = arg_ok and got.tobytes() == swapped.tobytes() and \
        np.ascontiguousarray(got.reshape(k, inner)[:, :cols]).tobytes() == ref.tobytes()
    b = 8  # one read and one write of every element
    out = {
        "metric": f"Gkeys/s, sort of float32 ({k}, 2^{log2n - 8}) along axis 0, 1 MI355X",
        "value": n / dt / 1e9, "unit": "Gkeys/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": f"sort along axis 0, float32, shape ({k}, {inner})",
                   "transposed_route_ms": dt_swapped * 1e3, "argsort_ms": dt_arg * 1e3,
                   "argsort_transposed_route_ms": dt_arg_swapped * 1e3},
        "parity_guard": "ok" if ok else "FAILED",
        "roofline": {"bound": "hbm", "kernel": "colsort_wave", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "achieved": b * n / dt / 1e9, "frac": b * n / dt / 1e9 / HBM_PEAK_GBS,
                     "traffic": float(8 * n) if log2n == 28 else None,
                     "note": "8 algorithmic bytes per key; traffic: FETCH_SIZE x2 + WRITE_SIZE x1 "
                             "of the column kernel equal the algorithmic bytes at 2^28"},
        "cpu_baseline": {"value": cpu, "unit": "Gkeys/s", "cores": 1, "kind": "port",
                         "sample": f"numpy stable sort along axis 0 of the first {cols} columns"},
    }
    print(json.dumps(out))
    return 0 if ok else 1


def run_sizes(args) -> int:
    """--workload sizes: single rows of 2^14 + 1 ... 2^21 elements (the sizes between the row
    kernels and the long rows of the radix path), int32 / float32 / int64, sort and stable
    argsort: one call timed alone with HIP events (median of 30) and back to back, the built-in
    plan beside the radix path asked for through misort_local_opts.  Not the headline."""
    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd._lib import Options
    from cunumeric_amd.config import to_core_dtype

    lib = _lib.load()
    dev = torch.device("cuda", 0)
    _lib.check(lib.misort_init())
    stream = torch.cuda.current_stream().cuda_stream
    rows, ok_all = [], True

    def one(dtype, n, argsort, opts, row_len=None):
        row_len = row_len or n
        rng = np.random.Generator(np.random.PCG64(1))
        if np.dtype(dtype).kind in "iu":
            ii = np.iinfo(dtype)
            a = rng.integers(ii.min, ii.max, n, dtype=dtype, endpoint=True)
        else:
            a = rng.random(n).astype(dtype)
        code = to_core_dtype(np.dtype(dtype))
        d_in = torch.from_numpy(a.view(np.uint8)).to(dev)
        d_out = torch.empty(n * 8, dtype=torch.uint8, device=dev)
        need = lib.misort_scratch_bytes_opts(code, n, row_len, int(argsort), 0, ctypes.byref(opts))
        scr = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        vo, io = (None, d_out.data_ptr()) if argsort else (d_out.data_ptr(), None)

        def call():
            _lib.check(lib.misort_local_opts(code, d_in.data_ptr(), vo, None, io, n, row_len, 1, 0, scr.data_ptr(),
                                             need, stream, ctypes.byref(opts)))

        for _ in range(5):
            call()
        torch.cuda.synchronize()
        ts = []
        for _ in range(30):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            call()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        t0 = time.perf_counter()
        for _ in range(30):
            call()
        torch.cuda.synchronize()
        b2b = (time.perf_counter() - t0) / 30 * 1e6
        a2 = a.reshape(-1, row_len)
        if argsort:
            ok = bool(np.array_equal(d_out.cpu().numpy().view(np.int64).reshape(a2.shape),
                                     np.argsort(a2, axis=1, kind="stable")))
        else:
            ok = d_out[: a.nbytes].cpu().numpy().tobytes() == np.sort(a2, axis=1, kind="stable").tobytes()
        return float(np.median(ts)), b2b, ok

    for dtype in (np.int32, np.float32, np.int64):
        for argsort in (False, True):
            for lg in range(14, 22):
                n = (1 << lg) + (1 if lg == 14 else 0)
                code = to_core_dtype(np.dtype(dtype))
                plan = _lib.describe_plan(code, n, n, argsort).split()[0]
                d = one(dtype, n, argsort, Options())
                r = one(dtype, n, argsort, Options(bucket_path=0, low_cardinality=0))
                ok_all = ok_all and d[2] and r[2]
                rows.append({"dtype": np.dtype(dtype).name, "argsort": argsort, "log2n": lg, "plan": plan,
                             "call_us": round(d[0], 1), "back_to_back_us": round(d[1], 1),
                             "radix_call_us": round(r[0], 1), "radix_back_to_back_us": round(r[1], 1)})
    # several rows side by side (rows too long for the row kernels, 2^20 elements in all)
    for dtype in (np.int32, np.int64):
        for argsort in (False, True):
            for n_rows in (2, 8, 32):
                row_len = (1 << 20) // n_rows
                code = to_core_dtype(np.dtype(dtype))
                plan = _lib.describe_plan(code, 1 << 20, row_len, argsort).split()[0]
                d = one(dtype, 1 << 20, argsort, Options(), row_len)
                r = one(dtype, 1 << 20, argsort, Options(bucket_path=0, low_cardinality=0), row_len)
                ok_all = ok_all and d[2] and r[2]
                rows.append({"dtype": np.dtype(dtype).name, "argsort": argsort, "log2n": 20, "rows": n_rows, "plan": plan,
                             "call_us": round(d[0], 1), "back_to_back_us": round(d[1], 1),
                             "radix_call_us": round(r[0], 1), "radix_back_to_back_us": round(r[1], 1)})
    out = {
        "metric": "microseconds per call, single rows of 2^14 .. 2^21 elements, 1 MI355X",
        "value": next(x["back_to_back_us"] for x in rows if x["dtype"] == "int32" and not x["argsort"] and x["log2n"] == 20),
        "unit": "us (int32 sort of 2^20, back to back)", "n_gpus": 1, "steps": 30, "warmup": 5,
        "ms_per_step": None, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic", "config": {"workload": "sizes sweep: uniform int32 / float32 / int64, sort and stable argsort"},
        "parity_guard": "ok" if ok_all else "FAILED", "sizes": rows,
    }
    print(json.dumps(out))
    return 0 if ok_all else 1


def gpu_library_baseline(workload: str, log2n: int):
    """The reference's device work for this workload (index fill + copy + CUB radix sort,
    src/cunumeric/sort/sort.cu:1694-1751 and cub_sort.cuh:36-189) served by hipCUB / rocPRIM on
    this GPU: oracle/hipcub_calls, a separate program run as a child process after the timed
    region.  A reported comparison, like cpu_baseline; None when the program is not built or
    has no case for the workload."""
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle", "hipcub_calls")
    if workload not in ("c1", "c2", "c4", "i64small") or not os.access(exe, os.X_OK):
        return None
    import subprocess
    try:
        r = subprocess.run([exe, workload, str(log2n), "10"], capture_output=True, text=True, timeout=300)
        d = json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:  # a baseline that does not run is reported, not fatal
        return {"value": None, "unit": "Gkeys/s", "kind": "hipcub", "error": str(e)[:200]}
    return {"value": d["Gkeys_per_s"], "unit": "Gkeys/s", "kind": "hipcub (rocPRIM) DeviceRadixSort, the "
            "reference's call sequence", "ms_median": d["ms_median"], "library_call_only_ms":
            d["library_call_only_ms"], "calls": d["calls"], "sample": f"2^{log2n} keys of the same "
            "distribution, generated on the device"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", choices=sorted(WORKLOADS) + ["ss", "uniq", "part", "sel", "axis", "sizes"], default="c2")
    ap.add_argument("--log2n", type=int, default=None)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calib-copy", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU local sort; it runs on exactly one GPU "
              "(--gpus 1). The multi-rank sample-sort exchange is not part of this build.",
              file=sys.stderr)
        return 2

    import torch

    from cunumeric_amd import _lib
    from cunumeric_amd.config import to_core_dtype

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _lib.load()  # raises if the HIP library is missing: no fallback
    if args.workload == "ss":
        return run_searchsorted(args)
    if args.workload == "uniq":
        return run_unique(args)
    if args.workload == "axis":
        return run_axis(args)
    if args.workload == "part":
        return run_partition(args)
    if args.workload == "sel":
        return run_select(args)
    if args.workload == "sizes":
        return run_sizes(args)
    dev = torch.device("cuda", 0)
    title, gen, def_log2n, argsort, row = WORKLOADS[args.workload]
    log2n = args.log2n if args.log2n is not None else def_log2n
    n = 1 << log2n
    if gen is None:
        a = make_c3(n // 256, 256)
    else:
        a = gen(n)
    host_api = row < 0
    row_len = n if row <= 0 else row
    k_bytes = a.dtype.itemsize
    v_bytes = 8 if argsort else 0
    code = to_core_dtype(a.dtype)
    from oracle import misort_oracle as oracle  # checker only

    stream = torch.cuda.current_stream().cuda_stream
    if host_api:
        import cunumeric_amd as num

        d_arr = num.array(a)
        result = {}

        def step():
            result["out"] = num.sort(d_arr, axis=0)

        plan = _lib.describe_plan(code, n, a.shape[0], False)
    else:
        d_in = torch.from_numpy(np.ascontiguousarray(a).reshape(-1).view(np.uint8)).to(dev)
        d_out = torch.empty(n * (8 if argsort else k_bytes), dtype=torch.uint8, device=dev)
        need = lib.misort_scratch_bytes(code, n, row_len, int(argsort), 0)
        scratch = torch.empty(need, dtype=torch.uint8, device=dev)
        plan = _lib.describe_plan(code, n, row_len, argsort)
        vo, io = (None, d_out.data_ptr()) if argsort else (d_out.data_ptr(), None)

        def step():
            _lib.check(lib.misort_local(code, d_in.data_ptr(), vo, None, io, n, row_len, 1, 0,
                                        scratch.data_ptr(), need, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    gkeys = n / (elapsed / args.steps) / 1e9

    # Where the sort ran by the upper key bytes first (plan upper_first_attempt): the same call
    # with all eight passes, for comparison (misort_options.upper_first = 0)
    eight_pass_ms = None
    if not host_api and "upper_first_attempt" in plan:
        from cunumeric_amd._lib import Options

        o8 = Options(upper_first=0)
        for _ in range(max(args.warmup, 1)):
            _lib.check(lib.misort_local_opts(code, d_in.data_ptr(), vo, None, io, n, row_len, 1, 0,
                                             scratch.data_ptr(), need, stream, ctypes.byref(o8)))
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            _lib.check(lib.misort_local_opts(code, d_in.data_ptr(), vo, None, io, n, row_len, 1, 0,
                                             scratch.data_ptr(), need, stream, ctypes.byref(o8)))
        torch.cuda.synchronize()
        eight_pass_ms = (time.perf_counter() - t1) / args.steps * 1e3
        step()  # (the output checked below is the default call's)
        torch.cuda.synchronize()

    # One call at a time: HIP events on the launch stream (torch's current stream is the one
    # handed to the library) from before the first launch to after the last kernel of the
    # call, the device idle before each call; median over the calls.
    n_ev = max(10, args.steps)
    ev_ms = []
    for _ in range(n_ev):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        step()
        e1.record()
        e1.synchronize()
        ev_ms.append(e0.elapsed_time(e1))
    call_ms = float(np.median(ev_ms))

    # quick parity guard on the timed output (the full oracle comparison lives in tests/):
    # argsort: the indices form a stable sorted order under the NumPy ordering;
    # sort: non-decreasing keys with the input's key checksum
    if host_api:
        got = np.asarray(result["out"])
        ok_shape = got.shape == a.shape
        ok_sorted = bool(np.all(got[:-1] <= got[1:]))
        ok_sum = bool(np.array_equal(oracle.to_key(got)[0].sum(axis=0, dtype=np.uint64),
                                     oracle.to_key(a)[0].sum(axis=0, dtype=np.uint64)))
        ok = ok_shape and ok_sorted and ok_sum
        if not ok:
            print(f"parity guard: shape {ok_shape} sorted {ok_sorted} checksum {ok_sum}", file=sys.stderr)
        del got
    elif argsort:
        idx = d_out.cpu().numpy().view(np.int64)
        words = oracle.to_key(a)
        keys = [w[idx] for w in words]
        hi = keys[-1]
        if len(keys) == 1:
            ok = bool(np.all(hi[:-1] <= hi[1:])) and bool(
                np.all((hi[:-1] != hi[1:]) | (idx[:-1] < idx[1:])))
        else:
            lo = keys[0]
            lt = (hi[:-1] < hi[1:]) | ((hi[:-1] == hi[1:]) & (lo[:-1] < lo[1:]))
            eq = (hi[:-1] == hi[1:]) & (lo[:-1] == lo[1:])
            ok = bool(np.all(lt | (eq & (idx[:-1] < idx[1:]))))
        del keys, idx, words
    else:
        got = d_out.cpu().numpy().view(a.dtype).reshape(-1, row_len)
        gk = oracle.to_key(got)[0]
        ok = bool(np.all(gk[:, :-1] <= gk[:, 1:]))
        ak = oracle.to_key(a.reshape(-1, row_len))[0]
        ok = ok and int(gk.sum(dtype=np.uint64)) == int(ak.sum(dtype=np.uint64))
        del got, gk, ak

    # per-kernel durations (HIP events around every launch, on the launch stream)
    kernels: dict = {}
    roofline = None
    if not host_api:
        max_k = 128
        kms = (ctypes.c_float * max_k)()
        kid = (ctypes.c_int * max_k)()
        nk = ctypes.c_int(0)
        reps = 10
        acc: dict = {}
        for _ in range(reps):
            _lib.check(lib.misort_local_profiled(code, d_in.data_ptr(), vo, None, io, n, row_len, 1, 0,
                                                 scratch.data_ptr(), need, stream, kms, kid, max_k,
                                                 ctypes.byref(nk)))
            for i in range(min(nk.value, max_k)):
                name = lib.misort_kernel_name(kid[i]).decode()
                acc.setdefault(name, []).append(kms[i])
        # avg_ms: median over the profiled calls of the mean duration of the kernel's launches
        # in one call.  Every launch sits between two events here, and the device idles for
        # the time an event takes between launches, so the sum over the kernels is an upper
        # bound of the call (call_ms, timed without the inner events, is the figure to use).
        # A radix pass over a digit that no key varies in is skipped on the device: its two
        # launches return at once, and so does, in large sorts, the last-pass form of the
        # scatter that is launched beside every middle pass in case the digits after it are
        # constant.  They are counted apart (launches whose median duration is
        # below a twentieth of the longest upsweep / scatter launch), so that the averages and
        # the roofline below are those of the passes that ran (P executed, not P planned).
        kernels = {}
        medians = {name: np.median(np.asarray(v, dtype=np.float64).reshape(reps, -1), axis=0)
                   for name, v in acc.items()}
        longest_scatter = max([m.max() for name, m in medians.items() if name.startswith("downsweep_")] or [0.0])
        # Long rows try the four-launch path first (plan low_cardinality_attempt): either its
        # count / scatter / bin sort kernels return at once (many distinct keys) or, if it went
        # through, every kernel of the radix path does.
        bucket_ms = medians["bucket_scatter"].max() if "bucket_scatter" in medians else 0.0
        attempt = "low_cardinality_attempt" in plan
        bucket_done = attempt and bucket_ms > 20 * longest_scatter
        bucket_dead = attempt and not bucket_done
        for name, v in acc.items():
            per_call = np.asarray(v, dtype=np.float64).reshape(reps, -1)
            per_launch = medians[name]
            if bucket_done and (name == "upsweep" or name.startswith("downsweep_")):
                ran = np.zeros_like(per_launch, dtype=bool)
            elif bucket_dead and name in ("bucket_count", "bucket_scatter", "bucket_sort"):
                ran = np.zeros_like(per_launch, dtype=bool)
            elif name == "upsweep":
                ran = per_launch >= 0.05 * per_launch.max()
            elif name.startswith("downsweep_"):
                # (with an attempt by the upper bytes first, plan upper_first_attempt, the launches
                # of the eight-pass sort follow and return at once, its first pass included)
                ran = per_launch >= 0.05 * longest_scatter
            else:
                ran = np.ones_like(per_launch, dtype=bool)
            if not ran.any():  # (every launch of this role returned at once)
                kernels[name] = {"launches_per_step": 0, "avg_ms": 0.0,
                                 "skipped_launches_per_step": int(per_launch.size),
                                 "skipped_avg_ms": float(per_launch.mean())}
                continue
            kernels[name] = {"launches_per_step": int(ran.sum()),
                             "avg_ms": float(np.median(per_call[:, ran].mean(axis=1)))}
            if not ran.all():
                kernels[name]["skipped_launches_per_step"] = int((~ran).sum())
                kernels[name]["skipped_avg_ms"] = float(per_launch[~ran].mean())
        all_ms = sum(k["avg_ms"] * k["launches_per_step"] +
                     k.get("skipped_avg_ms", 0.0) * k.get("skipped_launches_per_step", 0) for k in kernels.values())

        # roofline of the dominant kernel.  Radix plans: the downsweep scatter pass (all its
        # roles), algorithmic bytes per key per pass = first 2k+v, middle 2k+2v, last k+2v
        # (keys only: 2k).  Row plans: the row kernel reads and writes every key once.
        tot_bytes = tot_ms = 0.0
        n_launch = 0
        per_pass = {}
        dominant = "downsweep_kernel"
        for name, kk in kernels.items():
            if name.startswith("downsweep_"):
                b = algorithmic_bytes_per_key(k_bytes, v_bytes, name)
            elif name == "upper_first_fixup":
                b = k_bytes  # one read of the result's keys (the runs it sorts are a few per mille)
            elif name.startswith("rowsort_"):
                b, dominant = 2 * k_bytes + v_bytes, name
            elif name in ("count16_hist", "count16_fill"):
                # counting sort of 2-byte values: one read for the counts, one write
                b, dominant = k_bytes, "count16_hist"
            elif name.startswith("bucket_") and name != "bucket_plan":
                # medium rows: count reads the elements; scatter reads them and writes them with
                # 32-bit positions; the bin sort reads those and writes the result
                vp = 4 if argsort else 0
                if "strategy=bucket" in plan:
                    b = {"bucket_count": k_bytes, "bucket_scatter": 2 * k_bytes + vp,
                         "bucket_sort": k_bytes + vp + (v_bytes if argsort else k_bytes)}[name]
                    dominant = "bucket_sort"
                elif name == "bucket_sort":
                    continue  # (few distinct keys: nothing is left for the bin sort)
                else:
                    # few distinct keys: the scatter reads the elements and writes the result
                    b = {"bucket_count": k_bytes, "bucket_scatter": k_bytes + (v_bytes if argsort else k_bytes)}[name]
                    dominant = "bucket_scatter"
            else:
                continue
            l = kk["launches_per_step"]
            if l == 0:
                continue
            tot_bytes += b * n * l
            tot_ms += kk["avg_ms"] * l
            n_launch += l
            gbs = b * n / (kk["avg_ms"] * 1e-3) / 1e9
            per_pass[name] = {"bytes_per_key": b, "GB/s": gbs, "frac": gbs / HBM_PEAK_GBS}
        achieved = tot_bytes / (tot_ms * 1e-3) / 1e9 if tot_ms else 0.0
        n_up = kernels.get("upsweep", {}).get("launches_per_step", 0)
        if "upsweep" in kernels and n_up:
            # The first upsweep reads the keys.  A later one reads either the keys again or, where
            # the pass before left the digit side-band, one byte per key (plan side_band=1: every
            # later upsweep; side_band=2: decided per row on the device).  Each launch is priced
            # by what it read: with side_band=2 a launch that would exceed the device's pure read
            # rate (7 TB/s) at key width must have read bytes.
            side = 1 if "side_band=1" in plan else (2 if "side_band=2" in plan else 0)
            ups = medians["upsweep"]
            ran_up = ups >= 0.05 * ups.max()
            keys_ms, byte_ms = [], []
            for i, (ms_i, r_i) in enumerate(zip(ups, ran_up)):
                if not r_i:
                    continue
                bytes_read = i > 0 and (side == 1 or (side == 2 and k_bytes * n / (ms_i * 1e-3) / 1e9 > 7000.0))
                (byte_ms if bytes_read else keys_ms).append(float(ms_i))
            if keys_ms:
                gbs = k_bytes * n / (np.mean(keys_ms) * 1e-3) / 1e9
                per_pass["upsweep"] = {"bytes_per_key": k_bytes, "launches": len(keys_ms), "GB/s": gbs,
                                       "frac": gbs / HBM_PEAK_GBS}
            if byte_ms:
                gbs = n / (np.mean(byte_ms) * 1e-3) / 1e9
                per_pass["upsweep_side_band"] = {"bytes_per_key": 1, "launches": len(byte_ms), "GB/s": gbs,
                                                 "frac": gbs / HBM_PEAK_GBS}
        # whole sort: one histogram read + the passes (an LSD sort's minimum with a single
        # up-front histogram; this implementation reads the keys once more per pass)
        b_total = tot_bytes / n + (k_bytes if n_up else 0)
        if "strategy=bucket" in plan:
            # priced like the radix sort it stands in for (8-bit digits over the whole key: one
            # histogram read, P passes), so that the fraction compares with the radix path's
            P = k_bytes
            b_total = (k_bytes + 2 * k_bytes * P) if not argsort else \
                (4 * k_bytes + 3 * v_bytes + (P - 2) * (2 * k_bytes + 2 * v_bytes))
        traffic = None
        if args.workload == "c2" and log2n == 28:
            # from the rocprofv3 --pmc runs summarised in
            # profiles/downsweep_c2_f32_argsort_2p28_hbm_traffic.md (not measurable from here)
            traffic = C2_DOWNSWEEP_TRAFFIC_BYTES_PER_LAUNCH
        elif args.workload == "c3" and log2n == 28:
            # measured: the row kernel reads 2 GiB and writes 2 GiB (FETCH_SIZE x2, WRITE_SIZE x1)
            traffic = float(16 * n)
        roofline = {
            "bound": "hbm",
            "kernel": dominant,
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            # frac prices a launch with the ALGORITHMIC bytes (int64 positions in every pass);
            # frac_measured with the bytes the counters saw move (32-bit positions until the
            # last pass): the second one is the achieved HBM bandwidth
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "frac_measured": (traffic / (tot_ms / max(n_launch, 1) * 1e-3) / 1e9 / HBM_PEAK_GBS
                              if traffic else None),
            "algorithmic_bytes_per_launch": tot_bytes / max(n_launch, 1),
            "avg_launch_ms": tot_ms / max(n_launch, 1),
            "per_pass": per_pass,
            # the pass furthest from the roofline, and how many scatter passes ran (planned
            # passes whose digit no key varies in return at once and are not counted)
            "per_pass_min": (min(per_pass.items(), key=lambda kv: kv[1]["frac"])[0] if per_pass else None),
            "per_pass_min_frac": (min(v["frac"] for v in per_pass.values()) if per_pass else None),
            "passes_executed": sum(kk["launches_per_step"] for name, kk in kernels.items()
                                   if name.startswith("downsweep_")),
            # whole call: algorithmic bytes of all passes + one histogram read, over the time
            # of one call from its first launch to its last kernel's end (HIP events)
            "whole_sort": {"bytes_per_key": b_total, "call_ms": call_ms, "kernel_ms_sum": all_ms,
                           "GB/s": b_total * n / (call_ms * 1e-3) / 1e9,
                           "frac": b_total * n / (call_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        }

    # what a plain device copy reaches on this box (1 GiB read + 1 GiB written per copy)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    c0 = torch.cuda.Event(enable_timing=True)
    c1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    c0.record()
    for _ in range(10):
        dst.copy_(src)
    c1.record()
    c1.synchronize()
    copy_gbs = 10 * 2 * (1 << 30) / (c0.elapsed_time(c1) * 1e-3) / 1e9
    del src, dst

    shape = f"N=2^{log2n}" if row == 0 else f"{n // 256} x 256"
    out = {
        "metric": METRIC if args.workload == "c2" and log2n == 28 else f"Gkeys/s, {title}, 1 MI355X",
        "value": gkeys,
        "unit": "Gkeys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        # one call timed alone with HIP events (median of n), and its throughput
        "call_ms_median": call_ms,
        **({"ms_per_step_all_eight_passes": eight_pass_ms} if eight_pass_ms is not None else {}),
        "call_ms_n": n_ev,
        "value_per_call": n / (call_ms * 1e-3) / 1e9,
        "device_copy_GBs": copy_gbs,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {1: "u8", 2: "u16", 4: "u32", 8: "u64", 16: "u128"}[k_bytes],
        "data": "synthetic",
        "config": {"workload": f"{title}, {shape}", "plan": plan},
        "parity_guard": "ok" if ok else "FAILED",
        "kernels": kernels,
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
        flat = np.ascontiguousarray(a).reshape(-1)
        # 1-D: up to the whole headline input (a few seconds on 16 cores); rows: 2^25 elements
        sample_n = min(n, 1 << 28) if row == 0 else min(n, 1 << 25)
        cpu_row = sample_n if row == 0 else 256
        if host_api:
            out["cpu_baseline"] = {"value": None, "unit": "Gkeys/s", "cores": threads, "kind": "port",
                                   "sample": "see --workload c3"}
        else:
            out["cpu_baseline"] = cpu_baseline(flat[:sample_n], code, cpu_row, argsort, threads)
        lib_base = gpu_library_baseline(args.workload, log2n)
        if lib_base is not None:
            out["gpu_library_baseline"] = lib_base
    print(json.dumps(out))
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
