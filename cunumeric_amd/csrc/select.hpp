// Radix select: the key that a full sort would leave at position kth of every row, found
// without sorting.  One pass per key byte, most significant first:
//   select_hist_kernel   counts the current byte of the keys that still match the bytes
//                        fixed so far (one read of the row),
//   select_pick_kernel   finds the byte value whose bucket holds position kth, fixes it,
//                        and clears the counters for the next pass.
// After the last byte the pivot key is complete; partition / argpartition then run ONE
// three-way split pass (upsweep / downsweep with PART) around it.  The reference
// sorts completely for partition (cunumeric/deferred.py:3559-3578); NumPy only asks for
// the element at kth to be in its sorted place with nothing larger before it and nothing
// smaller after it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include "radix.hpp"

namespace misort {

constexpr int SEL_NT = 256;

// do the bytes of k above bit position `shift + 8` equal those of the prefix?
template <typename KeyT>
__device__ __forceinline__ bool select_matches(KeyT k, KeyT prefix, int shift)
{
  constexpr int BITS = sizeof(KeyT) * 8;
  if (shift + 8 >= BITS) return true;
  if constexpr (sizeof(KeyT) == 16) {
    if (shift + 8 >= 64) return ((k.hi ^ prefix.hi) >> (shift + 8 - 64)) == 0;
    return k.hi == prefix.hi && ((k.lo ^ prefix.lo) >> (shift + 8)) == 0;
  } else {
    return ((uint64_t)(k ^ prefix) >> (shift + 8)) == 0;
  }
}
template <typename KeyT>
__device__ __forceinline__ KeyT select_with_byte(KeyT prefix, uint32_t b, int shift)
{
  if constexpr (sizeof(KeyT) == 16) {
    if (shift >= 64) prefix.hi |= (uint64_t)b << (shift - 64);
    else prefix.lo |= (uint64_t)b << shift;
    return prefix;
  } else {
    return (KeyT)(prefix | (KeyT)((uint64_t)b << shift));
  }
}

// grid: rows * chunks_per_row; the chunk geometry is the one of the split pass that follows
template <typename KeyT>
__global__ void __launch_bounds__(SEL_NT)
select_hist_kernel(const KeyT* __restrict__ in, uint64_t row_len, uint64_t chunk_len,
                   uint32_t chunks_per_row, int xform, int shift, const KeyT* __restrict__ prefix,
                   unsigned long long* __restrict__ ghist)
{
  constexpr int NW = SEL_NT / 64, COPIES = 4;
  __shared__ __attribute__((aligned(16))) uint32_t h[NW * RADIX * COPIES];
  for (int i = threadIdx.x; i < NW * RADIX * COPIES; i += SEL_NT) h[i] = 0;
  __syncthreads();
  const uint32_t row = blockIdx.x / chunks_per_row, chunk = blockIdx.x % chunks_per_row;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t* my     = h + wave * (RADIX * COPIES) + (lane & (COPIES - 1));
  const KeyT pre   = prefix[row];
  const KeyT* base = in + (uint64_t)row * row_len;
  const uint64_t b0 = (uint64_t)chunk * chunk_len;
  uint64_t b1       = b0 + chunk_len;
  if (b1 > row_len) b1 = row_len;
  auto count = [&](KeyT raw) {
    const KeyT k = KeyOps<KeyT>::to_key(raw, xform);
    if (select_matches(k, pre, shift)) atomicAdd(&my[KeyOps<KeyT>::digit(k, shift) * COPIES], 1u);
  };
  // 16-byte loads where the row allows it
  constexpr int V = sizeof(KeyT) >= 16 ? 1 : 16 / sizeof(KeyT);
  struct alignas(16) Vec {
    KeyT v[V];
  };
  uint64_t i0 = b0;
  if (V > 1 && (reinterpret_cast<uintptr_t>(base + b0) & 15) == 0) {
    const uint64_t nvec = (b1 - b0) / V;
    const Vec* vb       = reinterpret_cast<const Vec*>(base + b0);
    if constexpr (sizeof(Vec) == 16) {
      stream_vectors<4>(vb, nvec, threadIdx.x, SEL_NT, [&](const Vec& r) {
#pragma unroll
        for (int e = 0; e < V; ++e) count(r.v[e]);
      });
    }
    i0 = b0 + nvec * V;
  }
  for (uint64_t i = i0 + threadIdx.x; i < b1; i += SEL_NT) count(base[i]);
  __syncthreads();
  for (int d = threadIdx.x; d < RADIX; d += SEL_NT) {
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const uint4 q = *reinterpret_cast<const uint4*>(&h[(w * RADIX + d) * COPIES]);
      c += q.x + q.y + q.z + q.w;
    }
    if (c) atomicAdd(&ghist[(uint64_t)row * RADIX + d], (unsigned long long)c);
  }
}

// grid: rows, RADIX threads.  kleft[row] = position of kth among the keys that match the prefix.
template <typename KeyT>
__global__ void __launch_bounds__(RADIX)
select_pick_kernel(KeyT* __restrict__ prefix, unsigned long long* __restrict__ kleft,
                   unsigned long long* __restrict__ ghist, int shift)
{
  __shared__ unsigned long long wave_tot[RADIX / 64];
  const uint32_t row = blockIdx.x;
  const int d = threadIdx.x, lane = d & 63, wave = d >> 6;
  unsigned long long* g      = ghist + (uint64_t)row * RADIX;
  const unsigned long long c = g[d];
  g[d]                       = 0;  // ready for the next pass
  const unsigned long long incl = wave_incl_scan(c, lane);
  if (lane == 63) wave_tot[wave] = incl;
  const unsigned long long k = kleft[row];
  __syncthreads();
  unsigned long long before = incl - c;
  for (int w = 0; w < wave; ++w) before += wave_tot[w];
  if (c != 0 && before <= k && k < before + c) {  // exactly one thread
    prefix[row] = select_with_byte(prefix[row], (uint32_t)d, shift);
    kleft[row]  = k - before;
  }
}

// grid-stride: prefix <- 0, kleft <- kth
template <typename KeyT>
__global__ void __launch_bounds__(256)
select_init_kernel(KeyT* __restrict__ prefix, unsigned long long* __restrict__ kleft, uint32_t rows,
                   unsigned long long kth)
{
  for (uint32_t r = blockIdx.x * 256 + threadIdx.x; r < rows; r += gridDim.x * 256) {
    prefix[r] = KeyT{};
    kleft[r]  = kth;
  }
}

}  // namespace misort
