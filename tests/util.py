"""Helpers shared by the tests: seeded inputs per dtype and a thin driver of the C ABI."""
from __future__ import annotations

import numpy as np

ALL_DTYPES = [
    np.bool_, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32,
    np.uint64, np.float16, np.float32, np.float64, np.complex64, np.complex128,
]


def random_array(dtype, n, rng, specials=True, narrow=False):
    """Seeded test data.  specials: sprinkle NaN (both signs, random payloads), +-0, +-inf
    into float / complex data.  narrow: few distinct values (heavy ties)."""
    dt = np.dtype(dtype)
    if dt == np.bool_:
        return rng.integers(0, 2, n).astype(dt)
    if dt.kind in "iu":
        ii = np.iinfo(dt)
        if narrow:
            lo, hi = max(ii.min, -3), min(ii.max, 3)
            return rng.integers(lo, hi, n, endpoint=True).astype(dt)
        return rng.integers(ii.min, ii.max, n, dtype=dt, endpoint=True)
    if dt.kind == "f":
        a = (rng.integers(-4, 4, n).astype(dt) if narrow else rng.standard_normal(n).astype(dt))
        if specials and n:
            u = np.dtype(f"u{dt.itemsize}")
            bits = a.view(u).copy()
            k = max(1, n // 16)
            mant_bits = {2: 10, 4: 23, 8: 52}[dt.itemsize]
            exp_all = ((1 << (dt.itemsize * 8 - 1 - mant_bits)) - 1) << mant_bits
            pos = rng.integers(0, n, k)
            payload = rng.integers(1, 1 << mant_bits, k, dtype=np.uint64)
            sign = rng.integers(0, 2, k, dtype=np.uint64) << np.uint64(dt.itemsize * 8 - 1)
            bits[pos] = (sign | np.uint64(exp_all) | payload).astype(u)
            a = bits.view(dt)
            a[rng.integers(0, n, k)] = -0.0
            a[rng.integers(0, n, k)] = 0.0
            a[rng.integers(0, n, max(1, k // 4))] = np.inf
            a[rng.integers(0, n, max(1, k // 4))] = -np.inf
        return a
    if dt.kind == "c":
        half = np.float32 if dt == np.complex64 else np.float64
        re = random_array(half, n, rng, specials, narrow=True)
        im = random_array(half, n, rng, specials, narrow)
        out = np.empty(n, dtype=dt)
        out.real, out.imag = re, im
        return out
    raise TypeError(dt)


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    return a.dtype == b.dtype and a.shape == b.shape and a.tobytes() == b.tobytes()


class Abi:
    """Calls misort_local with torch-owned device buffers; returns NumPy results."""

    def __init__(self):
        import torch

        from cunumeric_amd import _lib
        from cunumeric_amd.config import to_core_dtype

        self.torch = torch
        self._lib = _lib
        self.lib = _lib.load()
        self.to_code = to_core_dtype
        self.dev = torch.device("cuda", 0)
        # True: calls that name no options ask for the radix path where the library would pick
        # the four-launch path for medium rows (tests of the radix kernels on small arrays)
        self.force_radix = False
        # default of local_sort's early_last_bytes (None: the library's own limit)
        self.early_last_bytes = None

    def describe_plan(self, dtype, volume, sort_dim_size, argsort, options=None):
        if options is None and (self.force_radix or self.early_last_bytes is not None):
            from cunumeric_amd._lib import Options

            options = Options(early_last_min_bytes=-1 if self.early_last_bytes is None else self.early_last_bytes,
                              bucket_path=0 if self.force_radix else -1)
        return self._lib.describe_plan(self.to_code(np.dtype(dtype)), volume, sort_dim_size, argsort,
                                       options=options)

    def _up(self, a):
        t = self.torch
        a = np.ascontiguousarray(a)
        if a.nbytes == 0:
            return t.empty(16, dtype=t.uint8, device=self.dev)
        return t.from_numpy(a.reshape(-1).view(np.uint8).copy()).to(self.dev)

    def local_sort(self, values, sort_dim_size, argsort, indices_in=None, inplace=False,
                   index_offset=0, want_values=False, chunks=0, static=False, options=None,
                   early_last_bytes=None):
        """chunks != 0: misort_local_chunked with that chunk target; static: misort_local_static
        (the library's own scratch); options: a cunumeric_amd._lib.Options for misort_local_opts;
        early_last_bytes: that field of the options alone."""
        if early_last_bytes is None:
            early_last_bytes = self.early_last_bytes
        if options is None and not static and (early_last_bytes is not None or self.force_radix):
            from cunumeric_amd._lib import Options

            options = Options(target_chunks=chunks,
                              early_last_min_bytes=-1 if early_last_bytes is None else early_last_bytes,
                              bucket_path=0 if self.force_radix else -1)
        t = self.torch
        values = np.ascontiguousarray(values).reshape(-1)
        dt = values.dtype
        code = self.to_code(dt)
        volume = values.shape[0]
        d_in = self._up(values)
        d_vout = None
        if not argsort:
            d_vout = d_in if inplace else t.empty(max(values.nbytes, 16), dtype=t.uint8, device=self.dev)
        elif want_values:
            d_vout = t.empty(max(values.nbytes, 16), dtype=t.uint8, device=self.dev)
        d_iin = d_iout = None
        if argsort:
            if indices_in is not None:
                d_iin = self._up(np.ascontiguousarray(indices_in, dtype=np.int64))
                d_iout = d_iin if inplace else t.empty(max(volume * 8, 16), dtype=t.uint8, device=self.dev)
            else:
                d_iout = t.empty(max(volume * 8, 16), dtype=t.uint8, device=self.dev)
        stream = t.cuda.current_stream().cuda_stream
        ptr = lambda x: None if x is None else x.data_ptr()
        if static:
            rc = self.lib.misort_local_static(code, ptr(d_in), ptr(d_vout), ptr(d_iin), ptr(d_iout),
                                              volume, sort_dim_size, 1, index_offset, stream)
        elif options is not None:
            import ctypes

            need = self.lib.misort_scratch_bytes_opts(code, volume, sort_dim_size, int(argsort),
                                                      int(indices_in is not None), ctypes.byref(options))
            scratch = t.empty(max(need, 256), dtype=t.uint8, device=self.dev)
            rc = self.lib.misort_local_opts(code, ptr(d_in), ptr(d_vout), ptr(d_iin), ptr(d_iout),
                                            volume, sort_dim_size, 1, index_offset,
                                            scratch.data_ptr(), need, stream, ctypes.byref(options))
        elif chunks:
            need = self.lib.misort_scratch_bytes_chunked(code, volume, sort_dim_size, int(argsort),
                                                         int(indices_in is not None), chunks)
            scratch = t.empty(max(need, 256), dtype=t.uint8, device=self.dev)
            rc = self.lib.misort_local_chunked(code, ptr(d_in), ptr(d_vout), ptr(d_iin), ptr(d_iout),
                                               volume, sort_dim_size, 1, index_offset,
                                               scratch.data_ptr(), need, stream, chunks)
        else:
            need = self.lib.misort_scratch_bytes(code, volume, sort_dim_size, int(argsort),
                                                 int(indices_in is not None))
            scratch = t.empty(max(need, 256), dtype=t.uint8, device=self.dev)
            rc = self.lib.misort_local(code, ptr(d_in), ptr(d_vout), ptr(d_iin), ptr(d_iout), volume,
                                       sort_dim_size, 1, index_offset, scratch.data_ptr(), need, stream)
        self._lib.check(rc)
        t.cuda.synchronize()
        out_v = out_i = None
        if d_vout is not None:
            out_v = d_vout[: values.nbytes].cpu().numpy().view(dt).copy() if volume else np.empty(0, dt)
        if d_iout is not None:
            out_i = d_iout[: volume * 8].cpu().numpy().view(np.int64).copy() if volume else np.empty(0, np.int64)
        if argsort and want_values:
            return out_i, out_v
        return out_i if argsort else out_v
