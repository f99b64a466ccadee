// Bandwidth helpers around the sort kernels: gather by sorted position, dense 2-D
// transpose, and the patch that restores the original bit patterns of zeros and NaNs
// after a keys-only float sort.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include "launcher.hpp"

namespace misort {

// ---------------------------------------------------------------------------------------
// gather: out[r][j] = src[r][idx[r][j] - index_offset]
// (the sorted elements of an argsort; the reference instead lets CUB / Thrust carry a key
// copy, src/cunumeric/sort/sort.cu:1698, 1744-1751)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) gather_kernel(const T* __restrict__ src, T* __restrict__ out,
                                                     const int64_t* __restrict__ idx, uint64_t volume,
                                                     uint64_t row_len, int64_t index_offset)
{
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < volume;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t row = i / row_len;
    out[i]             = src[row * row_len + (uint64_t)(idx[i] - index_offset)];
  }
}

static void launch_gather(Launcher& L, int id, size_t elem_bytes, const void* src, void* out,
                          const int64_t* idx, size_t rows, size_t row_len, int64_t index_offset)
{
  const uint64_t volume = (uint64_t)rows * row_len;
  size_t blocks         = (volume + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  L.run(id, [&] {
    switch (elem_bytes) {
      case 1:
        hipLaunchKernelGGL(gather_kernel<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                           (const uint8_t*)src, (uint8_t*)out, idx, volume, (uint64_t)row_len,
                           index_offset);
        break;
      case 2:
        hipLaunchKernelGGL(gather_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                           (const uint16_t*)src, (uint16_t*)out, idx, volume, (uint64_t)row_len,
                           index_offset);
        break;
      case 4:
        hipLaunchKernelGGL(gather_kernel<uint32_t>, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                           (const uint32_t*)src, (uint32_t*)out, idx, volume, (uint64_t)row_len,
                           index_offset);
        break;
      case 8:
        hipLaunchKernelGGL(gather_kernel<uint64_t>, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                           (const uint64_t*)src, (uint64_t*)out, idx, volume, (uint64_t)row_len,
                           index_offset);
        break;
      default:
        hipLaunchKernelGGL(gather_kernel<u128>, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                           (const u128*)src, (u128*)out, idx, volume, (uint64_t)row_len,
                           index_offset);
        break;
    }
  });
}

// ---------------------------------------------------------------------------------------
// plain device copy (staging buffers of the single-pass and in-place cases back to the
// caller's array), in the widest unit both pointers and the size allow
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) copy_kernel(const T* __restrict__ src, T* __restrict__ dst, uint64_t n)
{
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

static void launch_copy(Launcher& L, int id, void* dst, const void* src, size_t bytes)
{
  if (bytes == 0) return;
  const uintptr_t mix = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes;
  const size_t unit   = (mix & 15) == 0 ? 16 : (mix & 7) == 0 ? 8 : (mix & 3) == 0 ? 4 : (mix & 1) == 0 ? 2 : 1;
  const uint64_t n    = bytes / unit;
  size_t blocks       = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  L.run(id, [&] {
#define MISORT_COPY_CASE(T)                                                                        \
  hipLaunchKernelGGL(copy_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, L.stream, (const T*)src, \
                     (T*)dst, n)
    switch (unit) {
      case 16: MISORT_COPY_CASE(u128); break;
      case 8: MISORT_COPY_CASE(uint64_t); break;
      case 4: MISORT_COPY_CASE(uint32_t); break;
      case 2: MISORT_COPY_CASE(uint16_t); break;
      default: MISORT_COPY_CASE(uint8_t); break;
    }
#undef MISORT_COPY_CASE
  });
}

// ---------------------------------------------------------------------------------------
// swap an axis with the last one: out[o][l][m][k] = in[o][k][m][l], 64 x 64 element tiles
// of the (k, l) plane staged through LDS so that both the reads (along l) and the writes
// (along k) are contiguous.  mid == 1 is a plain batched 2-D transpose.
// (the dense transposed copy made before a sort along a non-last axis,
// cunumeric/sort.py:47-83)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(1024)
swap_last_kernel(const T* __restrict__ in, T* __restrict__ out, uint32_t K, uint32_t M, uint32_t L,
                 uint32_t tiles_l, uint64_t planes)
{
  constexpr int TS = 64;
  __shared__ T tile[TS][TS + 1];
  const uint32_t tk = blockIdx.x / tiles_l, tl = blockIdx.x % tiles_l;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 16
  const uint32_t l  = tl * TS + tx;
  const uint32_t ko = tk * TS + tx;  // the fast index of the output
  const uint64_t plane = (uint64_t)K * M * L;
  // A tile that lies inside the array on both sides (all but the last row and column of
  // tiles) moves with four loads per thread asked for at once and no test per element: with a
  // test around every load the wait for one load was also the wait for all before it (C3
  // along axis 0: 0.945 -> 0.75 ms per copy of 2 GiB).
  const bool whole = (tk + 1) * TS <= K && (tl + 1) * TS <= L;
  // grid.y strides over the outer * mid planes (a launch dimension holds at most 65535)
  for (uint64_t om = blockIdx.y; om < planes; om += gridDim.y) {
    const uint64_t m = om % M, o = om / M;
    const T* src = in + o * plane + m * L;   // + k*M*L + l
    T* dst       = out + o * plane + m * K;  // + l*M*K + k
    if (whole) {
      T v[TS / 16];
#pragma unroll
      for (int i = 0; i < TS / 16; ++i)
        v[i] = load_streaming(&src[(uint64_t)(tk * TS + ty + 16 * i) * M * L + l]);
#pragma unroll
      for (int i = 0; i < TS / 16; ++i) tile[ty + 16 * i][tx] = v[i];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < TS / 16; ++i)
        dst[(uint64_t)(tl * TS + ty + 16 * i) * M * K + ko] = tile[tx][ty + 16 * i];
    } else {
      for (int j = ty; j < TS; j += 16) {
        const uint32_t k = tk * TS + j;
        if (k < K && l < L) tile[j][tx] = load_streaming(&src[(uint64_t)k * M * L + l]);
      }
      __syncthreads();
      for (int j = ty; j < TS; j += 16) {
        const uint32_t lo = tl * TS + j;
        if (lo < L && ko < K) dst[(uint64_t)lo * M * K + ko] = tile[tx][j];
      }
    }
    __syncthreads();
  }
}

static void launch_swap_last(Launcher& L_, int id, const void* in, void* out, size_t outer, size_t K,
                             size_t M, size_t L, size_t elem_bytes)
{
  const uint32_t tiles_k = (uint32_t)((K + 63) / 64), tiles_l = (uint32_t)((L + 63) / 64);
  const uint64_t planes  = (uint64_t)outer * M;
  const dim3 grid(tiles_k * tiles_l, (unsigned)(planes < 65535 ? planes : 65535));
  L_.run(id, [&] {
#define MISORT_SWAP_CASE(T)                                                                   \
  hipLaunchKernelGGL(swap_last_kernel<T>, grid, dim3(1024), 0, L_.stream, (const T*)in, (T*)out, \
                     (uint32_t)K, (uint32_t)M, (uint32_t)L, tiles_l, planes)
    switch (elem_bytes) {
      case 1: MISORT_SWAP_CASE(uint8_t); break;
      case 2: MISORT_SWAP_CASE(uint16_t); break;
      case 4: MISORT_SWAP_CASE(uint32_t); break;
      case 8: MISORT_SWAP_CASE(uint64_t); break;
      default: MISORT_SWAP_CASE(u128); break;
    }
#undef MISORT_SWAP_CASE
  });
}

// ---------------------------------------------------------------------------------------
// special elements of a keys-only float sort
//
// The radix key maps -0.0 and +0.0 to one key and every NaN to one key, and NumPy's stable
// sort keeps the original bit patterns of such ties in input order.  The first upsweep
// counts zeros / negative zeros / NaNs / negatives per wave sub-chunk; when a row holds a negative zero
// or a NaN, its zeros (resp. NaNs) are compacted in input order into a side buffer and
// copied over the zero run (resp. the NaN tail) of the sorted row.
//
// Per-row counters (unsigned long long[4]): {zeros, nans, negative zeros, negatives}.
// ---------------------------------------------------------------------------------------
constexpr int SP_ZERO = 0, SP_NAN = 1, SP_NEGZERO = 2, SP_NEG = 3;

// one block per row: exclusive scan of the per-sub-chunk {zero, nan} counts
__global__ void __launch_bounds__(256)
special_scan_kernel(unsigned long long* blk, const unsigned long long* rowctr,
                    uint32_t entries_per_row)
{
  const uint32_t row            = blockIdx.x;
  const unsigned long long* ctr = rowctr + (uint64_t)row * 4;
  if (ctr[SP_NEGZERO] == 0 && ctr[SP_NAN] == 0) return;
  __shared__ unsigned long long sz[256], sn[256];
  __shared__ unsigned long long carry[2];
  if (threadIdx.x == 0) carry[0] = carry[1] = 0;
  __syncthreads();
  unsigned long long* b = blk + (uint64_t)row * entries_per_row * 2;
  for (uint32_t base = 0; base < entries_per_row; base += 256) {
    const uint32_t e = base + threadIdx.x;
    unsigned long long z = 0, n = 0;
    if (e < entries_per_row) {
      z = b[2 * e];
      n = b[2 * e + 1];
    }
    sz[threadIdx.x] = z;
    sn[threadIdx.x] = n;
    __syncthreads();
    for (int s = 1; s < 256; s <<= 1) {
      unsigned long long tz = 0, tn = 0;
      if ((int)threadIdx.x >= s) {
        tz = sz[threadIdx.x - s];
        tn = sn[threadIdx.x - s];
      }
      __syncthreads();
      sz[threadIdx.x] += tz;
      sn[threadIdx.x] += tn;
      __syncthreads();
    }
    if (e < entries_per_row) {
      b[2 * e]     = carry[0] + sz[threadIdx.x] - z;
      b[2 * e + 1] = carry[1] + sn[threadIdx.x] - n;
    }
    __syncthreads();
    if (threadIdx.x == 255) {
      carry[0] += sz[255];
      carry[1] += sn[255];
    }
    __syncthreads();
  }
}

// same grid and wave sub-chunk ownership as the first upsweep.  into_sorted: `side` is the
// sorted output itself (the input is a different buffer and still intact after the sort):
// the zeros go straight over its zero run, which starts behind the negatives, the NaNs over
// its tail, and no patch kernel follows.
template <typename KeyT, int NT>
__global__ void __launch_bounds__(NT)
special_collect_kernel(const KeyT* __restrict__ in, KeyT* __restrict__ side,
                       const unsigned long long* __restrict__ blk,
                       const unsigned long long* __restrict__ rowctr, uint64_t row_len,
                       uint32_t chunks_per_row, uint64_t chunk, bool into_sorted)
{
  constexpr int NW          = NT / 64;
  const uint32_t row        = blockIdx.x / chunks_per_row;
  const uint32_t c          = blockIdx.x % chunks_per_row;
  const unsigned long long* ctr = rowctr + (uint64_t)row * 4;
  const bool do_zero        = ctr[SP_NEGZERO] != 0;
  const bool do_nan         = ctr[SP_NAN] != 0;
  if (!do_zero && !do_nan) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t sub   = chunk / NW;
  const uint64_t begin = (uint64_t)c * chunk + (uint64_t)wave * sub;
  uint64_t end         = begin + sub;
  if (end > row_len) end = row_len;
  const uint64_t e     = ((uint64_t)row * chunks_per_row + c) * NW + wave;
  unsigned long long zoff = blk[2 * e] + (into_sorted ? ctr[SP_NEG] : 0ull);
  unsigned long long noff = row_len - ctr[SP_NAN] + blk[2 * e + 1];
  const KeyT* rin = in + (uint64_t)row * row_len;
  KeyT* rside     = side + (uint64_t)row * row_len;
  using F         = FloatBits<KeyT>;
  for (uint64_t i0 = begin; i0 < end; i0 += 64) {
    const uint64_t i = i0 + lane;
    KeyT raw         = 0;
    bool isz = false, isn = false;
    if (i < end) {
      raw = rin[i];
      isn = float_is_nan(raw);
      isz = (KeyT)(raw & (KeyT)~F::SIGN) == 0;
    }
    const uint64_t mz = __ballot(isz), mn = __ballot(isn);
    const uint64_t lt = ((uint64_t)1 << lane) - 1;
    if (do_zero && isz) rside[zoff + __popcll(mz & lt)] = raw;
    if (do_nan && isn) rside[noff + __popcll(mn & lt)] = raw;
    zoff += __popcll(mz);
    noff += __popcll(mn);
  }
}

template <typename KeyT>
__global__ void __launch_bounds__(256)
special_patch_kernel(const KeyT* __restrict__ side, KeyT* __restrict__ out,
                     const unsigned long long* __restrict__ rowctr, uint64_t row_len,
                     uint32_t blocks_per_row)
{
  const uint32_t row            = blockIdx.x / blocks_per_row;
  const uint32_t b              = blockIdx.x % blocks_per_row;
  const unsigned long long* ctr = rowctr + (uint64_t)row * 4;
  const uint64_t rb             = (uint64_t)row * row_len;
  const uint64_t stride         = (uint64_t)blocks_per_row * 256;
  if (ctr[SP_NEGZERO] != 0) {
    const uint64_t neg = ctr[SP_NEG], nz = ctr[SP_ZERO];
    for (uint64_t j = (uint64_t)b * 256 + threadIdx.x; j < nz; j += stride)
      out[rb + neg + j] = side[rb + j];
  }
  if (ctr[SP_NAN] != 0) {
    const uint64_t nn = ctr[SP_NAN], start = row_len - nn;
    for (uint64_t j = (uint64_t)b * 256 + threadIdx.x; j < nn; j += stride)
      out[rb + start + j] = side[rb + start + j];
  }
}

}  // namespace misort
