// Long sorts of 8-byte keys, tried by the upper 32 to 48 bits first.
//
// Eight radix passes move every key eight times; the lower bytes only matter for keys that
// agree in the upper ones, and among 2^28 keys drawn from 64-bit integers a few thousand pairs
// agree in their upper 40 bits.  So the radix passes run over the upper four to
// six digits only (PassParams::digit_base; upper_first_digit0 below picks how many from the
// row length and the kind of key), which leaves the keys in order up to short runs of equal
// upper bits, and one more read of the result puts those runs right.  Float keys spend 12 of
// their upper bits on sign and exponent, which a few values share between all keys (2^27
// uniform doubles: a quarter of the keys in runs of equal upper 40 bits), so they keep more:
//
//   upper_first_plan_kernel   one workgroup sorts a sample of 8192 keys and lets the attempt go
//                             on only if no two sample keys agree in the upper bits while
//                             they differ below (small integers, clustered values: the runs
//                             would be long);
//   upper_first_fixup_kernel  every thread looks at its elements' neighbours in the result: a
//                             run of at most 16 elements with equal upper bits is sorted by
//                             the thread that holds its first element (by the whole key,
//                             stable); an element out of order inside a longer run calls the
//                             attempt off.
//
// Two words carry the decisions: flags[0] = go (the kernels of the attempt return at once if
// it is 0), flags[1] = done (set with go, cleared by the fix-up if a run was too long).  The
// kernels of the plain eight-pass sort follow on the stream and return at once if done is
// set: nothing comes back to the host.  The plain sort needs the input again, so the attempt
// is made only where the outputs do not alias the inputs.  No counterpart in the reference
// (cub::DeviceRadixSort runs all passes, src/cunumeric/sort/cub_sort.cuh:60-71).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bucket.hpp"
#include "lanes.hpp"

namespace misort {

// Digits left to the fix-up.  The passes keep the fewest upper bytes for which a row's keys,
// spread evenly, would have an expected run length of 1/32 or less: log2(row length) + 5 bits,
// plus what the key's upper bits do not spend on telling values apart (sign and exponent of a
// double: 12; the signs and exponents of both parts of a complex64 and the mantissa bits that
// its real part lacks: 15).  Runs of two are exchanged in passing, but a longer run costs its
// thread a dozen dependent reads and writes while its wavefront waits: with one key in sixteen
// in a run (2^28 int64 by their upper 32 bits) the fix-up took 2.5 ms instead of 0.55, as much
// as the pass it saved; at one in thirty-two (2^27) the sort is 8 % quicker with four passes.
// 2^27 int64: 32 bits (four passes); 2^28 int64: 40; rows of 2^20 doubles: 40; 2^28: 48.
static inline int upper_first_digit0(int xform, uint64_t row_len)
{
  const int spent = xform == XF_FLOAT ? 12 : xform == XF_COMPLEX ? 15 : 0;
  int need        = 5 + spent;
  while (need < 64 && (row_len >> (need - 5 - spent)) > 1) ++need;
  int bytes = (need + 7) / 8;
  if (bytes < 4) bytes = 4;
  if (bytes > 6) bytes = 6;
  return 8 - bytes;
}
constexpr int UF_RUN_LIMIT = 16;  // longest run the fix-up sorts
constexpr int UF_PLAN_NT   = 1024;
constexpr int UF_PLAN_IPT  = 8;   // 8192 sample keys
constexpr int UF_FIX_NT    = 256;
constexpr int UF_FIX_IPT   = 16;  // elements per thread of the fix-up

struct UpperFirstParams {
  const void* keys_in;         // plan: the elements as they came in
  uint64_t volume;             // elements in all rows
  uint64_t row_len;
  int xform;
  int low_bits;                // bits left to the fix-up (8 * upper_first_digit0)
  int mode;                    // 1: the sample decides; 2: go on whatever it says (tests)
  int rank_by_add;
  uint32_t* flags;             // [2]: go, done
  const uint32_t* prior_done;  // non-NULL: another attempt's "done" word; set = nothing left to do
  void* elems;                 // fix-up: the result's elements (complex: their keys), sorted by the upper bits
  int64_t* pos;                // fix-up: the payload that goes with them, or NULL
};

template <typename KeyT>
__global__ void __launch_bounds__(UF_PLAN_NT) upper_first_plan_kernel(UpperFirstParams p)
{
  static_assert(sizeof(KeyT) == 8, "8-byte keys");
  constexpr int NT = UF_PLAN_NT, IPT = UF_PLAN_IPT;
  __shared__ BlockSortSmem<KeyT, uint32_t, false, NT, IPT> sm;
  __shared__ unsigned long long ref;
  const int tid = threadIdx.x;
  if (p.prior_done && *p.prior_done) {  // the result is there already
    if (tid == 0) {
      p.flags[0] = 0u;
      p.flags[1] = 1u;
    }
    return;
  }
  if (p.mode == 2) {
    if (tid == 0) {
      p.flags[0] = 1u;
      p.flags[1] = 1u;
    }
    return;
  }
  const uint64_t n     = p.volume;
  const uint32_t S     = n < (uint64_t)NT * IPT ? (uint32_t)n : (uint32_t)(NT * IPT);
  const uint64_t span  = n / S > 0 ? n / S : 1;
  const KeyT* in       = reinterpret_cast<const KeyT*>(p.keys_in);
  const BlockSortGeom g = block_sort_geom<NT>(S);
  KeyT k[IPT];
  uint32_t nopay[1];
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const uint32_t e = g.wbase + i * 64;
    uint32_t h       = e * 0x9E3779B1u;
    h ^= h >> 15;
    h *= 0x85EBCA77u;
    h ^= h >> 13;
    uint64_t at = (uint64_t)e * n / S + h % span;  // (e < 2^13: no overflow below 2^51 elements)
    if (at >= n) at = n - 1;
    k[i] = ((uint32_t)i < g.R && e < S) ? KeyOps<KeyT>::to_key(in[at], p.xform) : KeyOps<KeyT>::max_key();
  }
  if (tid == 0) {
    ref     = (unsigned long long)k[0];
    sm.vary = 0;
  }
  __syncthreads();
  {
    const KeyT kr         = (KeyT)ref;
    unsigned long long vv = 0;
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      if ((uint32_t)i < g.R && g.wbase + i * 64 < S) {
        vv |= (unsigned long long)(KeyT)(k[i] ^ kr);
        sm.keys[g.wbase + i * 64] = k[i];
      }
    }
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) vv |= __shfl_xor(vv, sft, 64);
    if ((tid & 63) == 0 && vv) atomicOr(&sm.vary, vv);
    __syncthreads();
  }
  const unsigned long long vary = sm.vary;
  // in order of the upper bits is all that the question below needs
  const int lb                   = p.low_bits;
  const unsigned long long upper = vary & ~((1ull << lb) - 1);
  block_radix_sort<KeyT, uint32_t, false, NT, IPT>(sm.whist, sm.wave_tot, sm.keys, sm.pay, k, nopay, S, (KeyT)0, 64,
                                                   XF_UNSIGNED, p.rank_by_add, upper);
  int clustered = 0;
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const uint32_t e = (uint32_t)tid * IPT + j;
    if (e > 0 && e < S) {
      const unsigned long long a = (unsigned long long)sm.keys[e - 1], b = (unsigned long long)sm.keys[e];
      clustered |= ((a >> lb) == (b >> lb) && a != b) ? 1 : 0;
    }
  }
  clustered = __syncthreads_or(clustered);
  if (tid == 0) {
    const uint32_t go = clustered ? 0u : 1u;
    p.flags[0]        = go;
    p.flags[1]        = go;
  }
}

// One workgroup per stretch of UF_FIX_NT * UF_FIX_IPT elements of a row.
template <typename KeyT, bool HAS_POS>
__global__ void __launch_bounds__(UF_FIX_NT) upper_first_fixup_kernel(UpperFirstParams p, uint32_t chunks_per_row)
{
  if (p.flags[0] == 0) return;
  constexpr int NT = UF_FIX_NT, IPT = UF_FIX_IPT;
  const uint32_t row   = blockIdx.x / chunks_per_row;
  const uint32_t chunk = blockIdx.x % chunks_per_row;
  KeyT* el             = reinterpret_cast<KeyT*>(p.elems) + (uint64_t)row * p.row_len;
  int64_t* pos         = HAS_POS ? p.pos + (uint64_t)row * p.row_len : nullptr;
  const uint64_t n     = p.row_len;
  const int xf         = p.xform == XF_COMPLEX ? (int)XF_UNSIGNED : p.xform;  // (complex: keys as they are)
  auto key   = [&](KeyT e) { return KeyOps<KeyT>::to_key(e, xf); };
  const int lb = p.low_bits;
  auto upper   = [&](KeyT e) { return key(e) >> lb; };
  const uint64_t c0 = (uint64_t)chunk * (NT * IPT);
  // every thread's elements and their right neighbours, all loads in flight at once (a run that
  // another thread is sorting meanwhile may be seen half sorted: see below)
  KeyT ea[IPT], eb[IPT];
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const uint64_t i = c0 + (uint64_t)j * NT + threadIdx.x;
    ea[j]            = el[i < n ? i : n - 1];
    eb[j]            = el[i + 1 < n ? i + 1 : n - 1];
  }
  const int lane    = threadIdx.x & 63;
  uint32_t exchange = 0;  // bit j: elements i and i + 1 of slot j are a run of two in the wrong order
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const uint64_t i = c0 + (uint64_t)j * NT + threadIdx.x;
    const KeyT a = key(ea[j]), b = key(eb[j]);
    // the elements before and after the pair are the neighbouring lanes' (every lane takes
    // part in the exchange; the wavefront's first and last lane read theirs if they need them)
    KeyT before = __shfl_up(ea[j], 1, 64), after = __shfl_down(eb[j], 1, 64);
    if (i + 1 >= n) continue;  // (the last element of a row has no right neighbour; it may end a run)
    if ((a >> lb) != (b >> lb)) continue;
    const KeyT up = a >> lb;
    if (lane == 0 && i > 0) before = el[i - 1];
    if (lane == 63 && i + 2 < n) after = el[i + 2];
    const bool first = i == 0 || upper(before) != up;
    if (first && (i + 2 >= n || upper(after) != up)) {
      // a run of two, nearly all there are: in order, or exchanged below
      if (a > b) exchange |= 1u << j;
      continue;
    }
    // The upper bits of a place never change (runs are permuted inside themselves only), so
    // the extent of a run is safe to read while another thread sorts it; the whole keys of a
    // short run may be read half way through its sorting, which only matters for long runs,
    // that nobody touches.
    if (a > b) {
      // out of order: fine if the run is short (its first element's thread sorts it)
      uint64_t s = i, e = i + 2;
      while (s > 0 && i - s < (uint64_t)UF_RUN_LIMIT && upper(el[s - 1]) == up) --s;
      while (e < n && e - s <= (uint64_t)UF_RUN_LIMIT && upper(el[e]) == up) ++e;
      if (e - s > (uint64_t)UF_RUN_LIMIT) {
        p.flags[1] = 0u;  // a run too long to sort here: the plain passes run
        continue;
      }
    }
    if (!first) continue;  // not the first of its run
    uint64_t e = i + 2;
    while (e < n && e - i <= (uint64_t)UF_RUN_LIMIT && upper(el[e]) == up) ++e;
    if (e - i > (uint64_t)UF_RUN_LIMIT) continue;  // (in order already, or called off above)
    // insertion sort of [i, e) by the whole key; equal keys keep their order
    for (uint64_t x = i + 1; x < e; ++x) {
      const KeyT ex = el[x];
      const KeyT kx = key(ex);
      int64_t px    = 0;
      if constexpr (HAS_POS) px = pos[x];
      uint64_t y = x;
      while (y > i) {
        const KeyT ey = el[y - 1];
        if (key(ey) <= kx) break;
        el[y] = ey;
        if constexpr (HAS_POS) pos[y] = pos[y - 1];
        --y;
      }
      if (y != x) {
        el[y] = ex;
        if constexpr (HAS_POS) pos[y] = px;
      }
    }
  }
  // the runs of two that are in the wrong order: nobody else touches them, and the values read
  // at the start are theirs still.  All payload reads of a thread in flight together (one after
  // the other, each inside its slot's branch, they were most of the kernel's time).
  if (exchange) {
    int64_t p0[IPT], p1[IPT];
    if constexpr (HAS_POS) {
#pragma unroll
      for (int j = 0; j < IPT; ++j) {
        const uint64_t i = c0 + (uint64_t)j * NT + threadIdx.x;
        if ((exchange >> j) & 1u) {
          p0[j] = pos[i];
          p1[j] = pos[i + 1];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < IPT; ++j) {
      const uint64_t i = c0 + (uint64_t)j * NT + threadIdx.x;
      if ((exchange >> j) & 1u) {
        el[i]     = eb[j];
        el[i + 1] = ea[j];
        if constexpr (HAS_POS) {
          pos[i]     = p1[j];
          pos[i + 1] = p0[j];
        }
      }
    }
  }
}

}  // namespace misort
