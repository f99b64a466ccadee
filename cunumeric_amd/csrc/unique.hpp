// unique: the distinct elements of an array in sorted order.
//
// Replaces, for one GPU, the body of the UNIQUE task of the reference
// (src/cunumeric/set/unique.cu:150-180: copy, thrust::sort, thrust::unique; the NCCL tree
// merge that follows there combines the results of several ranks and has no counterpart
// here).  The sort is this library's values-only sort; what is left is a stream compaction
// of the sorted array:
//   unique_count_kernel    per block of 64 KB, how many elements start a run of equal keys,
//   unique_offsets_kernel  exclusive scan of those counts and the total (one workgroup),
//   unique_compact_kernel  every block writes its run heads at its offset.
// A block is 16 rows of 256 16-byte vectors; a thread takes one vector of every row (loads
// of a wavefront are contiguous) and the element before it, and run heads are numbered by
// (row, thread, element), which is their order in the array.  A block that is not whole, or
// an array that does not start on a 16-byte boundary, goes element by element.
// Two elements are equal when their sort keys are equal (-0 == +0); all NaNs (for complex:
// every element with a NaN part) count as one value, as in numpy.unique.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include "radix.hpp"

namespace misort {

constexpr int UNIQ_NT        = 256;
constexpr int UNIQ_ROWS      = 16;
constexpr int UNIQ_BLK_BYTES = UNIQ_NT * UNIQ_ROWS * 16;
// elements per block for elements of this size
constexpr uint64_t unique_block_elems(size_t elem_bytes) { return UNIQ_BLK_BYTES / elem_bytes; }

template <typename Raw>
__device__ __forceinline__ bool unique_is_nan(Raw r, int xform)
{
  if constexpr (sizeof(Raw) == 16) {
    return float_is_nan(r.lo) || float_is_nan(r.hi);
  } else if constexpr (sizeof(Raw) == 1) {
    return false;
  } else {
    if (xform == XF_FLOAT) return float_is_nan(r);
    if constexpr (sizeof(Raw) == 8) {
      if (xform == XF_COMPLEX) return float_is_nan((uint32_t)r) || float_is_nan((uint32_t)(r >> 32));
    }
    return false;
  }
}

// does element i of the sorted array start a run?
template <typename Raw>
__device__ __forceinline__ bool unique_is_head(const Raw* s, uint64_t i, int xform)
{
  if (i == 0) return true;
  const Raw cur = s[i], prev = s[i - 1];
  if (unique_is_nan(cur, xform)) return !unique_is_nan(prev, xform);
  return !key_eq(KeyOps<Raw>::to_key(cur, xform), KeyOps<Raw>::to_key(prev, xform));
}

// does cur start a run, given the element before it?
template <typename Raw>
__device__ __forceinline__ bool unique_differs(Raw prev, Raw cur, int xform)
{
  // the same bits are the same value, and integers with different bits differ; only floats
  // (-0 / +0, NaN patterns) need their keys
  if (key_eq(prev, cur)) return false;
  if (xform != XF_FLOAT && xform != XF_COMPLEX) return true;
  if (unique_is_nan(cur, xform)) return !unique_is_nan(prev, xform);
  return !key_eq(KeyOps<Raw>::to_key(cur, xform), KeyOps<Raw>::to_key(prev, xform));
}

template <typename Raw>
struct alignas(16) UniqueVec {
  Raw v[16 / sizeof(Raw)];
};

// the value the lane below holds (lane 0: unspecified)
template <typename Raw>
__device__ __forceinline__ Raw from_lane_below(Raw x)
{
  if constexpr (sizeof(Raw) <= 4) {
    return (Raw)__shfl_up((uint32_t)x, 1, 64);
  } else if constexpr (sizeof(Raw) == 8) {
    const uint32_t lo = __shfl_up((uint32_t)x, 1, 64), hi = __shfl_up((uint32_t)(x >> 32), 1, 64);
    return ((uint64_t)hi << 32) | lo;
  } else {
    Raw r;
    r.lo = from_lane_below<uint64_t>(x.lo);
    r.hi = from_lane_below<uint64_t>(x.hi);
    return r;
  }
}

// run heads among the elements of the vector at vector index iv, as a bit mask.  Adjacent
// lanes hold adjacent vectors, so the element before the vector is the last one of the lane
// below; only lane 0 reads it from memory.  Every lane of the wavefront must call this.
template <typename Raw>
__device__ __forceinline__ uint32_t unique_vector_heads(const Raw* s, uint64_t iv, const UniqueVec<Raw>& r,
                                                        int xform)
{
  constexpr int V = 16 / sizeof(Raw);
  Raw pred        = from_lane_below<Raw>(r.v[V - 1]);
  if ((threadIdx.x & 63) == 0 && iv > 0) pred = s[iv * V - 1];
  uint32_t m = iv == 0 ? 1u : (uint32_t)unique_differs(pred, r.v[0], xform);
#pragma unroll
  for (int e = 1; e < V; ++e) m |= (uint32_t)unique_differs(r.v[e - 1], r.v[e], xform) << e;
  return m;
}

template <typename Raw>
__device__ __forceinline__ bool unique_block_is_whole(const Raw* s, uint64_t n, uint64_t base)
{
  return (reinterpret_cast<uintptr_t>(s) & 15) == 0 && base + unique_block_elems(sizeof(Raw)) <= n;
}

template <typename Raw>
__global__ void __launch_bounds__(UNIQ_NT)
unique_count_kernel(const Raw* __restrict__ s, uint64_t n, int xform, unsigned long long* __restrict__ blk)
{
  constexpr int V        = 16 / sizeof(Raw);
  constexpr uint64_t BLK = unique_block_elems(sizeof(Raw));
  const uint64_t base    = (uint64_t)blockIdx.x * BLK;
  uint32_t c = 0;
  if (unique_block_is_whole(s, n, base)) {
    const UniqueVec<Raw>* vb = reinterpret_cast<const UniqueVec<Raw>*>(s);
    const uint64_t iv0       = base / V + threadIdx.x;
#pragma unroll
    for (int h = 0; h < UNIQ_ROWS; h += 8) {
      UniqueVec<Raw> r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) r[j] = load_streaming(&vb[iv0 + (uint64_t)(h + j) * UNIQ_NT]);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        c += __popc(unique_vector_heads(s, iv0 + (uint64_t)(h + j) * UNIQ_NT, r[j], xform));
    }
  } else {
    for (uint64_t i = base + threadIdx.x; i < base + BLK && i < n; i += UNIQ_NT)
      c += unique_is_head(s, i, xform);
  }
  __shared__ uint32_t wsum[UNIQ_NT / 64];
  c = wave_incl_scan_u32(c);
  if ((threadIdx.x & 63) == 63) wsum[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < UNIQ_NT / 64; ++w) t += wsum[w];
    blk[blockIdx.x] = t;
  }
}

// one workgroup: blk[b] <- number of run heads in the blocks before b; *count <- total
__global__ void __launch_bounds__(1024)
unique_offsets_kernel(unsigned long long* __restrict__ blk, uint64_t nblk, unsigned long long* __restrict__ count)
{
  __shared__ unsigned long long wave_tot[16];
  __shared__ unsigned long long carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (uint64_t b0 = 0; b0 < nblk; b0 += 1024) {
    const uint64_t b           = b0 + tid;
    const unsigned long long v = b < nblk ? blk[b] : 0ull;
    const unsigned long long incl = wave_incl_scan(v, lane);
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    unsigned long long before = carry;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    if (b < nblk) blk[b] = before + incl - v;
    __syncthreads();
    if (tid == 1023) carry = before + incl;
    __syncthreads();
  }
  if (tid == 0) *count = carry;
}

template <typename Raw>
__global__ void __launch_bounds__(UNIQ_NT)
unique_compact_kernel(const Raw* __restrict__ s, uint64_t n, int xform,
                      const unsigned long long* __restrict__ blk, Raw* __restrict__ out)
{
  constexpr int V        = 16 / sizeof(Raw);
  constexpr int NW       = UNIQ_NT / 64;
  constexpr uint64_t BLK = unique_block_elems(sizeof(Raw));
  const uint64_t base    = (uint64_t)blockIdx.x * BLK;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (unique_block_is_whole(s, n, base)) {
    static_assert(UNIQ_ROWS * NW == 64, "the cell scan below is one wavefront wide");
    // heads before (row j, wavefront w) inside the block: cell j * NW + w
    __shared__ uint32_t cell[UNIQ_ROWS * NW];
    const UniqueVec<Raw>* vb = reinterpret_cast<const UniqueVec<Raw>*>(s);
    const uint64_t iv0       = base / V + threadIdx.x;
    UniqueVec<Raw> r[UNIQ_ROWS];
    uint32_t heads[UNIQ_ROWS], before[UNIQ_ROWS];  // before: heads of the row in lower lanes
#pragma unroll
    for (int j = 0; j < UNIQ_ROWS; ++j) r[j] = load_streaming(&vb[iv0 + (uint64_t)j * UNIQ_NT]);
#pragma unroll
    for (int j = 0; j < UNIQ_ROWS; ++j) {
      heads[j]            = unique_vector_heads(s, iv0 + (uint64_t)j * UNIQ_NT, r[j], xform);
      const uint32_t c    = __popc(heads[j]);
      const uint32_t incl = wave_incl_scan_u32(c);
      before[j]           = incl - c;
      if (lane == 63) cell[j * NW + wave] = incl;
    }
    __syncthreads();
    if (wave == 0) {
      // exclusive prefix sum over the UNIQ_ROWS * NW = 64 cells in (row, wavefront) order
      const uint32_t v = cell[lane];
      cell[lane]       = wave_incl_scan_u32(v) - v;
    }
    __syncthreads();
    const unsigned long long at0 = blk[blockIdx.x];
#pragma unroll
    for (int j = 0; j < UNIQ_ROWS; ++j) {
      unsigned long long at = at0 + cell[j * NW + wave] + before[j];
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (heads[j] & (1u << e)) out[at++] = r[j].v[e];
    }
  } else {
    // thread t owns the consecutive elements base + t * IPT ..: run heads keep their order
    // (IPT from what the block holds: a short array is spread over all threads instead of
    // walked by the first few, element after element)
    const uint64_t left = n - base < BLK ? n - base : BLK;
    const uint64_t IPT  = (left + UNIQ_NT - 1) / UNIQ_NT;
    const uint64_t mine = base + (uint64_t)threadIdx.x * IPT;
    uint32_t c = 0;
    for (uint64_t i = mine; i < mine + IPT && i < n; ++i) c += unique_is_head(s, i, xform);
    __shared__ uint32_t wsum[NW];
    const uint32_t incl = wave_incl_scan_u32(c);
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    unsigned long long at = blk[blockIdx.x] + incl - c;
    for (int w = 0; w < wave; ++w) at += wsum[w];
    for (uint64_t i = mine; i < mine + IPT && i < n; ++i)
      if (unique_is_head(s, i, xform)) out[at++] = s[i];
  }
}

}  // namespace misort
