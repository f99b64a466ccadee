// searchsorted: for every query the insertion index into a sorted 1-D array.
//
// Replaces searchsorted_kernel_min / searchsorted_kernel_max of the reference
// (src/cunumeric/sort/searchsorted.cu:25-63: one cub::LowerBound / cub::UpperBound per
// query thread) for the case where one GPU holds the whole sorted array; the MIN / MAX
// reductions the reference needs to merge partial answers of several ranks
// (src/cunumeric/sort/searchsorted.cu:86-96, cunumeric/deferred.py:3511-3533) fall away.
//
// Comparisons run on the same unsigned keys as the sorts, so the answer agrees with the
// order those produce (NumPy's: NaN last, -0 == +0, complex lexicographic).  A workgroup
// first loads the keys of 64 KB worth of evenly spaced elements into LDS (16384 for 4-byte
// elements: 2^24 queries into 2^28 float32 take 3.83 ms, with 1024 entries 4.46 ms); a query searches that table, then
// only the one block of the array it points to.  Many queries are sorted first when the caller
// gives a workspace (searchsorted_sorted_kernel below): 1.18 ms for the same call.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include "radix.hpp"

namespace misort {

constexpr int SEARCH_NT  = 1024;
constexpr int SEARCH_TABLE_BYTES = 65536;  // all the LDS a workgroup may declare

template <typename Raw>
__global__ void __launch_bounds__(SEARCH_NT)
searchsorted_kernel(const Raw* __restrict__ a, uint64_t n, const Raw* __restrict__ v, uint64_t m,
                    int xform, int left, int64_t* __restrict__ out)
{
  constexpr int SEARCH_SPL = SEARCH_TABLE_BYTES / sizeof(Raw);  // table entries
  __shared__ Raw table[SEARCH_SPL];
  const uint64_t step = (n + SEARCH_SPL - 1) / SEARCH_SPL;  // elements per block, >= 1 when n > 0
  const uint32_t nblk = n == 0 ? 0u : (uint32_t)((n + step - 1) / step);
  // table[b] = key of the last element of block b
  for (uint32_t b = threadIdx.x; b < nblk; b += SEARCH_NT) {
    uint64_t last = (uint64_t)(b + 1) * step;
    if (last > n) last = n;
    table[b] = KeyOps<Raw>::to_key(a[last - 1], xform);
  }
  __syncthreads();

  // does an element with key `e` lie at or after the insertion point of key `q`?
  auto beyond = [&](Raw e, Raw q) { return left ? !key_lt(e, q) : key_lt(q, e); };

  for (uint64_t j = (uint64_t)blockIdx.x * SEARCH_NT + threadIdx.x; j < m;
       j += (uint64_t)gridDim.x * SEARCH_NT) {
    const Raw q = KeyOps<Raw>::to_key(v[j], xform);
    // first block whose last element is beyond the insertion point
    uint32_t lo = 0, hi = nblk;
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (beyond(table[mid], q)) hi = mid; else lo = mid + 1;
    }
    uint64_t ans = n;
    if (lo < nblk) {
      // first element of that block that is beyond it (the last one is)
      uint64_t l = (uint64_t)lo * step, h = (uint64_t)(lo + 1) * step;
      if (h > n) h = n;
      --h;  // known to be beyond
      while (l < h) {
        const uint64_t mid = (l + h) >> 1;
        if (beyond(KeyOps<Raw>::to_key(a[mid], xform), q)) h = mid; else l = mid + 1;
      }
      ans = l;
    }
    out[j] = (int64_t)ans;
  }
}

// The same for queries that arrive in ascending order, with where[j] the position query j
// came from (the queries sorted by this library with their positions): random queries into
// an array far larger than the caches are bound by one cache-line fetch per probe, sorted
// ones share their lines.  A workgroup takes per_block consecutive queries.  Two wavefronts
// first find the insertion points of the first and of the last of them (64-ary search: the
// lanes sample the range, a ballot picks the block, five rounds for 2^28 elements); every
// other answer lies between those two, so the table in LDS samples only that stretch of the
// array (a 2^-11 th of it for 2^24 queries), and a query needs a few probes inside one or two
// lines after the table.  The answer goes to out[where[j]].
template <typename Raw>
__global__ void __launch_bounds__(SEARCH_NT)
searchsorted_sorted_kernel(const Raw* __restrict__ a, uint64_t n, const Raw* __restrict__ v, uint64_t m,
                           int xform, int left, int64_t* __restrict__ out,
                           const int64_t* __restrict__ where, uint64_t per_block)
{
  constexpr int SEARCH_SPL = SEARCH_TABLE_BYTES / sizeof(Raw) - 64;  // table entries
  __shared__ Raw table[SEARCH_SPL];
  __shared__ unsigned long long bounds[2];
  auto beyond = [&](Raw e, Raw q) { return left ? !key_lt(e, q) : key_lt(q, e); };
  const uint64_t j0 = (uint64_t)blockIdx.x * per_block;
  if (j0 >= m) return;
  const uint64_t j1 = j0 + per_block < m ? j0 + per_block : m;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  if (wave < 2) {
    // insertion point of one query over the whole array; invariant: it lies in [lo, hi], and
    // hi is n or the index of an element known to be beyond it
    const Raw q = KeyOps<Raw>::to_key(v[wave == 0 ? j0 : j1 - 1], xform);
    uint64_t lo = 0, hi = n;
    while (hi > lo) {
      const uint64_t len  = hi - lo;
      const uint64_t step = (len + 63) / 64;
      const bool active   = (uint64_t)lane * step < len;
      uint64_t last       = ((uint64_t)lane + 1) * step;
      if (last > len) last = len;
      const bool b        = active ? beyond(KeyOps<Raw>::to_key(a[lo + last - 1], xform), q) : true;
      const uint64_t mask = __ballot(b);
      const int f         = mask ? __builtin_ctzll(mask) : 64;
      if (f == 64 || (uint64_t)f * step >= len) {  // no sampled element is beyond: the answer is hi
        lo = hi;
        break;
      }
      uint64_t fl = ((uint64_t)f + 1) * step;
      if (fl > len) fl = len;
      hi = lo + fl - 1;  // that element is beyond
      lo = lo + (uint64_t)f * step;
    }
    if (lane == 0) bounds[wave] = lo;
  }
  __syncthreads();
  const uint64_t L = bounds[0], H = bounds[1];
  const uint64_t len  = H - L;  // every answer of this workgroup lies in [L, H]
  const uint64_t step = len ? (len + SEARCH_SPL - 1) / SEARCH_SPL : 1;
  const uint32_t nblk = (uint32_t)((len + step - 1) / step);
  // table[b] = key of the last element of block b of a[L .. H)
  for (uint32_t b = threadIdx.x; b < nblk; b += SEARCH_NT) {
    uint64_t last = (uint64_t)(b + 1) * step;
    if (last > len) last = len;
    table[b] = KeyOps<Raw>::to_key(a[L + last - 1], xform);
  }
  __syncthreads();
  for (uint64_t j = j0 + threadIdx.x; j < j1; j += SEARCH_NT) {
    const Raw q = KeyOps<Raw>::to_key(v[j], xform);
    uint32_t lo = 0, hi = nblk;
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (beyond(table[mid], q)) hi = mid; else lo = mid + 1;
    }
    uint64_t ans = H;
    if (lo < nblk) {
      uint64_t l = (uint64_t)lo * step, h = (uint64_t)(lo + 1) * step;
      if (h > len) h = len;
      --h;  // known to be beyond
      while (l < h) {
        const uint64_t mid = (l + h) >> 1;
        if (beyond(KeyOps<Raw>::to_key(a[L + mid], xform), q)) h = mid; else l = mid + 1;
      }
      ans = L + l;
    }
    out[(uint64_t)where[j]] = (int64_t)ans;
  }
}

}  // namespace misort
