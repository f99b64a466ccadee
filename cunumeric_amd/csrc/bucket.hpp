// Sort of rows of a few ten thousand to about two million elements in four launches: sample
// -> count -> scatter -> sort the bins.  It serves the sizes where the radix path's two
// launches per digit are mostly launch and start-up time (the reference's own benchmark sorts
// 10^6 elements, examples/sort.py:110-123; the calls replaced are the same ones,
// src/cunumeric/sort/cub_sort.cuh:60-71, 120-143 and thrust_sort.cuh:61-66).
//
//   bucket_plan_kernel     one workgroup draws 16 samples per bin at scattered places, sorts
//                          their keys in LDS and keeps every 16th as a splitter (at most 255);
//   bucket_count_kernel    every chunk counts its keys per bin: bin 2j holds the keys strictly
//                          between splitters j-1 and j, bin 2j+1 the keys equal to splitter j, so
//                          a value that fills half the array fills a bin that needs no sorting;
//   bucket_scatter_kernel  every chunk moves its elements to their bins, in input order (chunks
//                          in order, elements of a chunk in order): the pass is stable;
//   bucket_sort_kernel     one workgroup per bin: the bin in registers, an LSD radix sort over
//                          the key bits that can differ inside the bin (from its two splitters),
//                          permuting through LDS; the result goes straight to the output.
// Splitters from a sorted sample make the bins even whatever the distribution of the keys
// (with 16 samples per bin one four times the average is a 1e-18 event), and equal keys take no
// room in the bins that are sorted.  A bin that does not fit the registers all the same is
// sorted by its workgroup through global memory (bucket_sort_long): slow, and correct.
// Elements travel as they came in (the key is derived where it is needed), so a stable sort
// keeps the bit patterns of zeros and NaNs in input order with no patching afterwards; complex
// keys, which are not cheap to derive, travel as keys with the elements as their payload.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "lanes.hpp"
#include "radix.hpp"

namespace misort {

constexpr int BK_SLOTS      = 256;  // splitter table: 255 splitters at most, padded with the largest key
constexpr int BK_BINS       = 512;
constexpr int BK_OVERSAMPLE = 16;   // samples per splitter interval
constexpr int BK_OVERSAMPLE_MAX = 32;  // for rows whose bins average more than 5/12 of what the bin sort holds
constexpr int BK_PLAN_NT    = 1024;  // the planning workgroup sorts up to 1024 * 4 sample keys
constexpr int BK_PLAN_IPT   = 4;  // 4096 sample keys (8 for the 8192 of BK_OVERSAMPLE_MAX)
constexpr int BK_COUNT_NT   = 1024;
constexpr int BK_NT         = 1024;  // scatter and bin sort

struct BucketParams {
  const void* keys_in;   // the row, elements as they came in
  const void* pay_in;    // PAY_I64: the caller's payload; else unused (positions are made up)
  void* keys_out;        // sorted elements, or NULL
  void* pay_out;         // int64 payload / positions (+ index_offset), or NULL
  void* buf_keys[2];     // scratch: the row in bin order ([1]: second buffer for long bins)
  void* buf_pay[2];      // scratch: its payload (u32 positions or int64)
  void* splitters;       // KeyT[BK_SLOTS], ascending keys, written by the plan kernel
  uint32_t* chunk_hist;  // [n_chunks][BK_BINS]
  uint32_t* slab_tot;    // [n_slabs][BK_BINS], cleared by the plan kernel
  uint32_t* bin_start;   // [BK_BINS + 1] first position of every bin, written by chunk 0 of the scatter
  unsigned long long* chunk_range;  // [n_chunks][2] smallest and largest key of every chunk (count kernel)
  unsigned long long* key_range;    // [2] smallest and largest key of the row (chunk 0 of the scatter)
  // Several rows of the same length are sorted side by side: the second launch dimension is the
  // row, and every pointer above (but flags) is the first row's: row r has its elements at
  // r * n, its splitters at r * BK_SLOTS, its slab totals at r * n_slabs * BK_BINS, its chunk
  // counts at r * n_chunks * BK_BINS, its bin starts at r * (BK_BINS + 1), its chunks' key ranges
  // at r * n_chunks * 2 and its own at r * 2.
  uint32_t n;            // elements in a row
  uint32_t n_split;      // splitters in use
  uint32_t oversample;   // samples per bin (BK_OVERSAMPLE_MAX at most)
  uint32_t tile, tiles_per_chunk, n_chunks, chunks_per_slab, n_slabs;
  uint32_t cap;          // longest bin sorted in registers
  int64_t index_offset;
  int xform;             // of the elements in keys_in
  int keys_travel;       // 1: the scatter writes keys (complex), 0: the elements themselves
  int rank_by_add;
  int direct_equal;      // 1: the scatter writes the bins of equal keys straight to the outputs
                         // (outputs do not alias the inputs); 0: the bin sort copies them
  // Long rows, which the radix path serves: this path is tried first where the keys take few
  // distinct values (every value a bin of its own, filled by the scatter; nothing left to
  // sort), and the radix kernels that follow return at once if it went through.
  //   flags[0]  set by the plan kernel: go on (the sample holds at most 255 distinct keys, which
  //             then are the splitters; or attempt == 2, which tries with any sample)
  //   flags[1]  set by the scatter: done (no bin that needs sorting is longer than cap);
  //             the bin sort runs if it is set, the radix kernels if it is not
  // NULL: the path runs unconditionally.
  uint32_t* flags;
  int attempt;           // 0: not an attempt; 1: only with few distinct sample keys; 2: always
};

// The kernels' view of one row: every pointer of the parameters moved to that row (the
// parameters themselves stay untouched in the kernel's argument segment).
template <typename KeyT, typename PayT>
struct BucketRow {
  const KeyT* keys_in;
  const int64_t* pay_in;
  KeyT* keys_out;
  int64_t* pay_out;
  KeyT* buf_keys0;
  KeyT* buf_keys1;
  PayT* buf_pay0;
  PayT* buf_pay1;
  KeyT* splitters;
  uint32_t* slab_tot;
  uint32_t* chunk_hist;
  uint32_t* bin_start;
  unsigned long long* chunk_range;
  unsigned long long* key_range;
  __device__ __forceinline__ BucketRow(const BucketParams& p, uint32_t row)
  {
    const size_t e0 = (size_t)row * p.n;
    keys_in    = static_cast<const KeyT*>(p.keys_in) + e0;
    pay_in     = p.pay_in ? static_cast<const int64_t*>(p.pay_in) + e0 : nullptr;
    keys_out   = p.keys_out ? static_cast<KeyT*>(p.keys_out) + e0 : nullptr;
    pay_out    = p.pay_out ? static_cast<int64_t*>(p.pay_out) + e0 : nullptr;
    buf_keys0  = static_cast<KeyT*>(p.buf_keys[0]) + e0;
    buf_keys1  = static_cast<KeyT*>(p.buf_keys[1]) + e0;
    buf_pay0   = p.buf_pay[0] ? static_cast<PayT*>(p.buf_pay[0]) + e0 : nullptr;
    buf_pay1   = p.buf_pay[1] ? static_cast<PayT*>(p.buf_pay[1]) + e0 : nullptr;
    splitters  = static_cast<KeyT*>(p.splitters) + (size_t)row * BK_SLOTS;
    slab_tot   = p.slab_tot + (size_t)row * p.n_slabs * BK_BINS;
    chunk_hist = p.chunk_hist + (size_t)row * p.n_chunks * BK_BINS;
    bin_start  = p.bin_start + (size_t)row * (BK_BINS + 1);
    chunk_range = p.chunk_range + (size_t)row * p.n_chunks * 2;
    key_range   = p.key_range + (size_t)row * 2;
  }
};

// Rank of this lane's key among the keys with the same digit value that the wavefront has
// ranked so far (earlier calls, lower lanes of this one); my_hist: the wavefront's counters in
// LDS.  by_add: one returning add, which relies on the LDS serving the lanes of one instruction
// that hit the same word in ascending lane order (the library checks that once per GPU);
// otherwise the lanes with the same value find each other with one ballot per digit bit.
// Every lane of the wavefront must be active; lanes with valid == false hold no key.
template <int BITS>
__device__ __forceinline__ uint32_t wave_rank(uint32_t* my_hist, uint32_t d, bool valid, int by_add)
{
  if (by_add) return valid ? atomicAdd(&my_hist[d], 1u) : 0u;
  uint64_t peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < BITS; ++b) {
    const bool bit    = (d >> b) & 1u;
    const uint64_t bl = __ballot(bit);
    peers &= bit ? bl : ~bl;
  }
  const uint32_t below =
    __builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
  const uint32_t cnt = (uint32_t)__popcll(peers);
  // the lowest peer adds the group's size; LDS runs a wavefront's operations in order, so the
  // read that follows sees the counter after this call and no later one
  if (valid && below == 0) atomicAdd(&my_hist[d], cnt);
  const uint32_t after = __hip_atomic_load(&my_hist[d], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  return after - cnt + below;
}

// ---------------------------------------------------------------------------------------
// splitter table in LDS: the sorted splitters and the same keys laid out as a search tree
// ---------------------------------------------------------------------------------------
template <typename KeyT>
struct SplitterTable {
  KeyT sorted[BK_SLOTS];  // [j] = splitter j; unused slots and [255] hold the largest key
  KeyT tree[BK_SLOTS];    // node j (1 .. 255) of a complete binary tree over sorted[0 .. 254]
};

template <typename KeyT, int NT>
__device__ __forceinline__ void load_splitters(SplitterTable<KeyT>& t, const KeyT* spl)
{
  for (int j = threadIdx.x; j < BK_SLOTS; j += NT) t.sorted[j] = spl[j];
  __syncthreads();
  for (int j = threadIdx.x; j < BK_SLOTS; j += NT) {
    if (j == 0) {
      t.tree[0] = t.sorted[0];  // never read
    } else {
      const int l   = 31 - __builtin_clz((unsigned)j);
      const int pos = j - (1 << l);
      t.tree[j]     = t.sorted[((2 * pos + 1) << (7 - l)) - 1];
    }
  }
  __syncthreads();
}

// Bin of a key: twice the number of splitters below it, plus one if it equals the next one.
template <typename KeyT>
__device__ __forceinline__ uint32_t bin_of(const SplitterTable<KeyT>& t, KeyT k)
{
  uint32_t j = 1;
#pragma unroll
  for (int l = 0; l < 8; ++l) j = 2 * j + (k > t.tree[j] ? 1u : 0u);
  j -= BK_SLOTS;
  return 2 * j + (t.sorted[j] == k ? 1u : 0u);
}

// ---------------------------------------------------------------------------------------
// radix sort of up to NT * IPT elements held by a workgroup, least significant digit first.
// The len elements lie in rows of 64; every wavefront owns R consecutive rows, R just large
// enough that the NT / 64 wavefronts cover them all (a short bin is spread over all wavefronts:
// a wavefront alone on its SIMD issues an instruction only every dozen clocks).  Element
// e = (wave * R + i) * 64 + lane sits in slot i < R of its thread.  Sorts by the bits
// [0, nbits) of to_key(element, xform) - base.
// ---------------------------------------------------------------------------------------
template <typename KeyT, typename PayT, bool HAS_PAY, int NT, int IPT>
struct BlockSortSmem {
  uint32_t whist[(NT / 64) * RADIX];
  uint32_t wave_tot[NT / 64];
  unsigned long long vary;
  __attribute__((aligned(16))) KeyT keys[NT * IPT];
  __attribute__((aligned(16))) PayT pay[HAS_PAY ? NT * IPT : 1];
};

struct BlockSortGeom {
  uint32_t R;      // rows per wavefront: a power of two
  uint32_t wbase;  // element of this thread's slot 0
};
template <int NT>
__device__ __forceinline__ BlockSortGeom block_sort_geom(uint32_t len)
{
  BlockSortGeom g;
  const uint32_t rows = (len + 63) / 64;
  const uint32_t r    = (rows + NT / 64 - 1) / (NT / 64);
  g.R                 = r <= 1 ? 1u : 1u << (32 - __builtin_clz(r - 1));
  g.R                 = (uint32_t)__builtin_amdgcn_readfirstlane((int)g.R);
  g.wbase             = (threadIdx.x >> 6) * g.R * 64 + (threadIdx.x & 63);
  return g;
}

// the passes for R = RR rows per wavefront: straight-line code over the RR slots (rows that
// lie beyond the elements have no valid lane and do nothing)
// SHARED_LDS: skeys and spay are the same memory (16384 elements of 12 or 16 bytes do not fit
// the LDS side by side); the payload then follows the keys through it in a second step.
// check_lo > 0 (8-byte keys): the caller has left the passes below bit check_lo out of `vary`;
// the return value says whether this thread saw two neighbours of the result that agree in
// the bits from check_lo up and differ below, in which case the result is not in order yet
// and the caller runs all passes (from any order, and stable: equal keys never trade places).
template <typename KeyT, typename PayT, bool HAS_PAY, int NT, int IPT, int RR, bool SHARED_LDS = false>
__device__ __forceinline__ bool block_radix_sort_rows(uint32_t* whist, uint32_t* wave_tot, KeyT* skeys,
                                                      PayT* spay, KeyT (&el)[IPT],
                                                      PayT (&pay)[HAS_PAY ? IPT : 1], uint32_t len, KeyT base,
                                                      int nbits, int xform, int by_add, unsigned long long vary,
                                                      int check_lo = 0)
{
  static_assert(NT % RADIX == 0 && RR <= IPT, "whole groups of one thread per digit value");
  constexpr int NW  = NT / 64;
  constexpr int NG  = NT / RADIX;  // thread groups, each covering all digit values
  constexpr int WPG = NW / NG;     // wavefronts whose counters a group rewrites
  const int tid        = threadIdx.x;
  const int lane       = tid & 63;
  const int wave       = tid >> 6;
  const uint32_t wbase = (uint32_t)wave * (RR * 64) + lane;
  uint32_t* my_hist    = whist + wave * RADIX;
  const uint32_t dv    = tid & (RADIX - 1);
  const int grp        = wave / (RADIX / 64);
  const bool is_float  = xform == XF_FLOAT;
  const KeyT flip      = xform == XF_SIGNED ? (KeyT)((KeyT)1 << (sizeof(KeyT) * 8 - 1)) : (KeyT)0;
  for (int i = tid; i < NW * RADIX; i += NT) whist[i] = 0;  // (a pass leaves them cleared for the next)
  int last_shift = -1;
  bool bad       = false;
  if constexpr (sizeof(KeyT) == 8) {
    if (check_lo)
      for (int sh = 0; sh < nbits; sh += RADIX_BITS)
        if ((vary >> sh) & (RADIX - 1)) last_shift = sh;
  }
  for (int shift = 0; shift < nbits; shift += RADIX_BITS) {
    if (((vary >> shift) & (RADIX - 1)) == 0) continue;  // (same in every thread)
    uint32_t d[RR], r[RR];
    if (is_float) {
#pragma unroll
      for (int i = 0; i < RR; ++i) d[i] = KeyOps<KeyT>::digit((KeyT)(float_to_key(el[i]) - base), shift);
    } else {
#pragma unroll
      for (int i = 0; i < RR; ++i) d[i] = KeyOps<KeyT>::digit((KeyT)((KeyT)(el[i] ^ flip) - base), shift);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RR; ++i) r[i] = wave_rank<RADIX_BITS>(my_hist, d[i], wbase + i * 64 < len, by_add);
    __syncthreads();
    // every thread takes digit value dv and the wavefronts of its group; all groups add up the
    // value's count over every wavefront and scan the counts over the digit values for themselves
    uint32_t count = 0, before = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == grp * WPG) before = count;
      count += whist[w * RADIX + dv];
    }
    const uint32_t incl = wave_incl_scan_u32(count);
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    {
      uint32_t off = incl - count + before;
      for (int w = grp * (RADIX / 64); w < wave; ++w) off += wave_tot[w];
      uint32_t* mine = whist + grp * WPG * RADIX + dv;
#pragma unroll
      for (int w = 0; w < WPG; ++w) {
        const uint32_t c = mine[w * RADIX];
        mine[w * RADIX]  = off;
        off += c;
      }
    }
    __syncthreads();
    uint32_t q[RR];
#pragma unroll
    for (int i = 0; i < RR; ++i) q[i] = my_hist[d[i]] + r[i];
#pragma unroll
    for (int i = 0; i < RR; ++i) {
      if (wbase + i * 64 < len) {
        skeys[q[i]] = el[i];
        if constexpr (HAS_PAY && !SHARED_LDS) spay[q[i]] = pay[i];
      }
    }
    __syncthreads();
    for (int i = tid; i < NW * RADIX; i += NT) whist[i] = 0;  // (read for the last time before the barrier)
#pragma unroll
    for (int i = 0; i < RR; ++i) {
      if (wbase + i * 64 < len) {
        el[i] = skeys[wbase + i * 64];
        if constexpr (HAS_PAY && !SHARED_LDS) pay[i] = spay[wbase + i * 64];
      }
    }
    if constexpr (sizeof(KeyT) == 8) {
      if (shift == last_shift) {  // (only with check_lo, in the last pass that runs)
#pragma unroll
        for (int i = 0; i < RR; ++i) {
          const uint32_t e = wbase + i * 64;
          if (e > 0 && e < len) {
            const KeyT pe = skeys[e - 1];
            const KeyT ka = (KeyT)((is_float ? float_to_key(pe) : (KeyT)(pe ^ flip)) - base);
            const KeyT kb = (KeyT)((is_float ? float_to_key(el[i]) : (KeyT)(el[i] ^ flip)) - base);
            bad |= (ka >> check_lo) == (kb >> check_lo) && ka != kb;
          }
        }
      }
    }
    if constexpr (HAS_PAY && SHARED_LDS) {
      __syncthreads();  // (every key has been read back)
#pragma unroll
      for (int i = 0; i < RR; ++i)
        if (wbase + i * 64 < len) spay[q[i]] = pay[i];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < RR; ++i)
        if (wbase + i * 64 < len) pay[i] = spay[wbase + i * 64];
      // (the next pass writes keys only after two more barriers)
    }
  }
  return bad;
}

// xform: XF_UNSIGNED, XF_SIGNED or XF_FLOAT (complex keys are transformed before they get here)
template <typename KeyT, typename PayT, bool HAS_PAY, int NT, int IPT>
__device__ __forceinline__ bool block_radix_sort(uint32_t* whist /* (NT / 64) * RADIX */,
                                                 uint32_t* wave_tot /* NT / 64 */,
                                                 KeyT* skeys /* NT * IPT */, PayT* spay /* NT * IPT */,
                                                 KeyT (&el)[IPT], PayT (&pay)[HAS_PAY ? IPT : 1],
                                                 uint32_t len, KeyT base, int nbits, int xform, int by_add,
                                                 unsigned long long vary = ~0ull /* bits in which keys differ */,
                                                 int check_lo = 0)
{
  const uint32_t R = block_sort_geom<NT>(len).R;
#define MISORT_BK_ROWS(RR)                                                                                          \
  return block_radix_sort_rows<KeyT, PayT, HAS_PAY, NT, IPT, RR>(whist, wave_tot, skeys, spay, el, pay, len, base, \
                                                                 nbits, xform, by_add, vary, check_lo)
  if (R == 1) MISORT_BK_ROWS(1);
  else if (R == 2) MISORT_BK_ROWS(2);
  else if (R == 4) MISORT_BK_ROWS(4);
  else if constexpr (IPT >= 8) {
    if (R == 8) MISORT_BK_ROWS(8);
    else if constexpr (IPT >= 16) MISORT_BK_ROWS(16);
  }
#undef MISORT_BK_ROWS
  return false;
}

// The bits that 8-byte keys are sorted by first: the 40 or more most significant of those that
// can differ, from a digit boundary up (`vary`; bits [0, nbits) of key - base).  Two of 4096 or 16384 keys that agree in all
// of them and differ below are rare (uniform doubles: one sample in 250), so the passes
// below mostly never run.  Returns the first bit kept (0: all passes run anyway).
__device__ __forceinline__ int upper_bits_first(unsigned long long vary, unsigned long long& vary_top)
{
  vary_top     = vary;
  const int hb = vary ? 63 - __builtin_clzll(vary) : 0;
  if (hb < 40) return 0;
  const int lo = 8 * ((hb + 1 - 40) / 8);  // (40 to 47 bits stay)
  vary_top     = vary & ~((1ull << lo) - 1);
  return vary_top != vary ? lo : 0;
}

// ---------------------------------------------------------------------------------------
// plan: splitters from a sorted sample; also clears the slab totals of the count kernel
// ---------------------------------------------------------------------------------------
template <typename KeyT, int IPT = BK_PLAN_IPT>
__global__ void __launch_bounds__(BK_PLAN_NT) bucket_plan_kernel(BucketParams p)
{
  constexpr int NT = BK_PLAN_NT;
  __shared__ BlockSortSmem<KeyT, uint32_t, false, NT, IPT> sm;
  const int tid = threadIdx.x;
  const BucketRow<KeyT, uint32_t> r(p, blockIdx.x);  // one workgroup per row (the payload is not touched)
  for (uint32_t i = tid; i < p.n_slabs * BK_BINS; i += NT) r.slab_tot[i] = 0;
  // sample e of S comes from its own stretch of n / S elements, at a place inside it that a hash
  // of e picks (evenly spaced places would meet periodic data at the same phase every time)
  const uint32_t S     = (p.n_split + 1) * p.oversample;  // <= NT * IPT
  const uint32_t span  = p.n / S > 0 ? p.n / S : 1;
  const KeyT* in       = r.keys_in;
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
    uint64_t pos = (uint64_t)e * p.n / S + h % span;
    if (pos >= p.n) pos = p.n - 1;
    k[i] = ((uint32_t)i < g.R && e < S) ? KeyOps<KeyT>::to_key(in[pos], p.xform) : KeyOps<KeyT>::max_key();
  }
  // which bits vary over the sample: passes over a digit that is the same in every sample key
  // move nothing and are left out (the upper bytes of small integers, the low bytes of
  // floats that hold integers)
  {
    __shared__ unsigned long long ref;
    if (tid == 0) {
      ref     = (unsigned long long)k[0];  // sample 0
      sm.vary = 0;
    }
    __syncthreads();
    const KeyT kr         = (KeyT)ref;
    unsigned long long vv = 0;
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      if ((uint32_t)i < g.R && g.wbase + i * 64 < S) {
        vv |= (unsigned long long)(KeyT)(k[i] ^ kr);
        sm.keys[g.wbase + i * 64] = k[i];  // (if no pass runs at all, the sample is sorted as it is)
      }
    }
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) vv |= __shfl_xor(vv, sft, 64);
    if ((tid & 63) == 0 && vv) atomicOr(&sm.vary, vv);
    __syncthreads();
  }
  // (8-byte keys: by the upper 40 varying bits first, by all of them only if that left two
  // sample keys in the wrong order: three passes less, 3-6 us)
  unsigned long long vary_top = sm.vary;
  int lo                      = 0;
  if constexpr (sizeof(KeyT) == 8) lo = upper_bits_first(sm.vary, vary_top);
  const bool bad = block_radix_sort<KeyT, uint32_t, false, NT, IPT>(sm.whist, sm.wave_tot, sm.keys, sm.pay, k, nopay,
                                                                   S, (KeyT)0, (int)sizeof(KeyT) * 8, XF_UNSIGNED,
                                                                   p.rank_by_add, vary_top, lo);
  if (lo && __syncthreads_or(bad ? 1 : 0))  // (lo is the same in every thread)
    block_radix_sort<KeyT, uint32_t, false, NT, IPT>(sm.whist, sm.wave_tot, sm.keys, sm.pay, k, nopay, S, (KeyT)0,
                                                     (int)sizeof(KeyT) * 8, XF_UNSIGNED, p.rank_by_add, sm.vary);
  // the sorted sample is still in sm.keys; splitter t = the last sample of stretch t
  KeyT* spl = r.splitters;
  if (p.attempt) {
    // an attempt on a long row: if the sample holds at most 255 distinct keys, those are the
    // splitters, each with a bin of equal keys behind it
    __shared__ uint32_t wave_heads[NT / 64];
    const int lane = tid & 63, wave = tid >> 6;
    constexpr int PER = IPT;  // sample keys [PER * tid, PER * tid + PER) per thread
    uint32_t heads = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const uint32_t e = (uint32_t)tid * PER + j;
      heads += (e < S && (e == 0 || sm.keys[e] != sm.keys[e - 1])) ? 1u : 0u;
    }
    const uint32_t incl = wave_incl_scan_u32(heads);
    if (lane == 63) wave_heads[wave] = incl;
    __syncthreads();
    uint32_t first = incl - heads, total = 0;
    for (int w = 0; w < NT / 64; ++w) {
      if (w < wave) first += wave_heads[w];
      total += wave_heads[w];
    }
    const bool few = total <= (uint32_t)(BK_SLOTS - 1);
    if (few) {
      for (uint32_t t = tid; t < BK_SLOTS; t += NT) spl[t] = KeyOps<KeyT>::max_key();
      __syncthreads();  // (the padding is in place before the distinct keys go over it)
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const uint32_t e = (uint32_t)tid * PER + j;
        if (e < S && (e == 0 || sm.keys[e] != sm.keys[e - 1])) spl[first++] = sm.keys[e];
      }
    }
    if (tid == 0) {
      p.flags[0] = (few || p.attempt == 2) ? 1u : 0u;
      p.flags[1] = 0u;
    }
    if (few) return;
  }
  for (uint32_t t = tid; t < BK_SLOTS; t += NT)
    spl[t] = t < p.n_split ? sm.keys[(t + 1) * p.oversample - 1] : KeyOps<KeyT>::max_key();
}

// ---------------------------------------------------------------------------------------
// count: keys per bin of every chunk, added up per slab of chunks
// ---------------------------------------------------------------------------------------
template <typename KeyT, bool TRACK = true>
__global__ void __launch_bounds__(BK_COUNT_NT) bucket_count_kernel(BucketParams p)
{
  constexpr int NT = BK_COUNT_NT, NW = NT / 64;
  __shared__ SplitterTable<KeyT> tab;
  __shared__ uint32_t hist[NW * BK_BINS];
  if (p.flags && p.flags[0] == 0) return;  // an attempt that the plan kernel called off
  const BucketRow<KeyT, uint32_t> r(p, blockIdx.y);
  const int tid = threadIdx.x, wave = tid >> 6;
  __shared__ unsigned long long wmin[NW], wmax[NW];
  for (int i = tid; i < NW * BK_BINS; i += NT) hist[i] = 0;
  load_splitters<KeyT, NT>(tab, r.splitters);
  const uint32_t chunk = blockIdx.x;
  const uint64_t clen  = (uint64_t)p.tiles_per_chunk * p.tile;
  const uint64_t b0    = (uint64_t)chunk * clen;
  const uint64_t b1    = b0 + clen < p.n ? b0 + clen : p.n;
  const KeyT* in       = r.keys_in;
  uint32_t* my         = hist + wave * BK_BINS;
  // (rounds of U independent loads per thread; the next round is asked for before this one is
  // searched, U searches side by side)
  constexpr int U = 4;
  auto fetch = [&](KeyT (&raw)[U], uint64_t i0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t i = i0 + (uint64_t)u * NT + tid;
      raw[u]           = in[i < b1 ? i : b0];
    }
  };
  // (the smallest and the largest key of the chunk as well: the first and the last bin have no
  // splitter on their outer side, and the bin sort takes its bits from the bounds of a bin;
  // a lane past the end holds the chunk's first key again)
  // (not on a long row's attempt, whose bins that need sorting are few and short: the bounds
  // are then the smallest and the largest key there is)
  // (TRACK = false: a compare more per key in this loop cost the count of 2^28 keys 0.16 ms)
  KeyT kmin = TRACK ? KeyOps<KeyT>::max_key() : (KeyT)0, kmax = TRACK ? (KeyT)0 : KeyOps<KeyT>::max_key();
  auto consume = [&](const KeyT (&raw)[U], uint64_t i0) {
    uint32_t b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const KeyT k = KeyOps<KeyT>::to_key(raw[u], p.xform);
      if constexpr (TRACK) {
        kmin = k < kmin ? k : kmin;
        kmax = k > kmax ? k : kmax;
      }
      b[u] = bin_of(tab, k);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + (uint64_t)u * NT + tid < b1) atomicAdd(&my[b[u]], 1u);
  };
  {
    KeyT ra[U], rb[U];
    uint64_t i0 = b0;
    if (i0 < b1) fetch(ra, i0);
    while (i0 < b1) {
      const uint64_t i1 = i0 + (uint64_t)U * NT, i2 = i1 + (uint64_t)U * NT;
      if (i1 < b1) fetch(rb, i1);
      consume(ra, i0);
      if (i1 >= b1) break;
      if (i2 < b1) fetch(ra, i2);
      consume(rb, i1);
      i0 = i2;
    }
  }
  {
    unsigned long long mn = (unsigned long long)kmin, mx = (unsigned long long)kmax;
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) {
      const unsigned long long a = __shfl_xor(mn, sft, 64), b = __shfl_xor(mx, sft, 64);
      mn = a < mn ? a : mn;
      mx = b > mx ? b : mx;
    }
    if ((tid & 63) == 0) {
      wmin[wave] = mn;
      wmax[wave] = mx;
    }
  }
  __syncthreads();
  if (tid < 64) {  // (one wavefront: the NW partial results in its first lanes)
    static_assert(NW <= 64 && (NW & (NW - 1)) == 0, "a power of two of partial results");
    unsigned long long mn = wmin[tid & (NW - 1)], mx = wmax[tid & (NW - 1)];
#pragma unroll
    for (int sft = NW / 2; sft > 0; sft >>= 1) {
      const unsigned long long a = __shfl_xor(mn, sft, 64), b = __shfl_xor(mx, sft, 64);
      mn = a < mn ? a : mn;
      mx = b > mx ? b : mx;
    }
    if (tid == 0) {
      r.chunk_range[2 * chunk]     = mn;
      r.chunk_range[2 * chunk + 1] = mx;
    }
  }
  uint32_t* out  = r.chunk_hist + (uint64_t)chunk * BK_BINS;
  uint32_t* slab = r.slab_tot + (uint64_t)(chunk / p.chunks_per_slab) * BK_BINS;
  for (int b = tid; b < BK_BINS; b += NT) {
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) c += hist[w * BK_BINS + b];
    out[b] = c;
    if (c) atomicAdd(&slab[b], c);
  }
}

// ---------------------------------------------------------------------------------------
// scatter: the elements of every chunk to their bins, in input order
// ---------------------------------------------------------------------------------------
template <typename KeyT, int PAY, int IPT>
__global__ void __launch_bounds__(BK_NT) bucket_scatter_kernel(BucketParams p)
{
  constexpr int NT = BK_NT, NW = NT / 64, TILE = NT * IPT;
  using PayT = typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type;
  constexpr bool HAS_PAY = PAY != PAY_NONE;
  static_assert(TILE <= 65535, "the staged bin of an element is a 16-bit word");
  __shared__ SplitterTable<KeyT> tab;
  __shared__ uint32_t whist[NW * BK_BINS];
  __shared__ uint32_t bin_base[BK_BINS];  // first staged slot of every bin in the tile
  __shared__ uint32_t gpos[BK_BINS];      // where the chunk's next element of every bin goes
  __shared__ uint32_t wave_tot[BK_BINS / 64];
  __shared__ __attribute__((aligned(16))) KeyT skeys[TILE];
  __shared__ __attribute__((aligned(16))) PayT spay[HAS_PAY ? TILE : 1];
  __shared__ uint16_t sbin[TILE];

  if (p.flags && p.flags[0] == 0) return;  // an attempt that the plan kernel called off
  const BucketRow<KeyT, PayT> r(p, blockIdx.y);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t wbase = (uint32_t)wave * (64 * IPT) + lane;
  const uint32_t chunk = blockIdx.x;
  const KeyT* in       = r.keys_in;
  const uint32_t tile0 = chunk * p.tiles_per_chunk;
  const uint32_t tiles = (p.n + TILE - 1) / TILE;
  uint32_t tile_end    = tile0 + p.tiles_per_chunk;
  if (tile_end > tiles) tile_end = tiles;
  // the first tile is asked for before anything else: the splitters and the counts of the
  // chunks before this one arrive meanwhile
  KeyT el[IPT];
  PayT pv[HAS_PAY ? IPT : 1];
  auto load_tile = [&](uint32_t t) {
    const uint32_t t0    = t * TILE;
    const uint32_t valid = p.n - t0 < (uint32_t)TILE ? p.n - t0 : (uint32_t)TILE;
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t e = wbase + i * 64;
      el[i]            = in[t0 + (e < valid ? e : 0u)];
      if constexpr (PAY == PAY_I64) pv[i] = r.pay_in[t0 + (e < valid ? e : 0u)];
      if constexpr (PAY == PAY_IDX32) pv[i] = t0 + e;
    }
  };
  if (tile0 < tile_end) load_tile(tile0);
  __shared__ unsigned long long wmin[NW], wmax[NW];  // chunk 0: the row's smallest and largest key
  load_splitters<KeyT, NT>(tab, r.splitters);

  // ---- where this chunk's elements of every bin start: the bins before (all chunks), the
  // same bin in the slabs before this chunk's and in the chunks before it inside its slab
  {
    // chunk 0 also works out the row's smallest and largest key from the chunks', for the bin
    // sort of the first and the last bin
    if (chunk == 0) {
      unsigned long long mn = ~0ull, mx = 0ull;
      for (uint32_t c = tid; c < p.n_chunks; c += NT) {
        const unsigned long long a = r.chunk_range[2 * c], b = r.chunk_range[2 * c + 1];
        mn = a < mn ? a : mn;
        mx = b > mx ? b : mx;
      }
#pragma unroll
      for (int sft = 32; sft > 0; sft >>= 1) {
        const unsigned long long a = __shfl_xor(mn, sft, 64), b = __shfl_xor(mx, sft, 64);
        mn = a < mn ? a : mn;
        mx = b > mx ? b : mx;
      }
      if (lane == 0) {
        wmin[wave] = mn;
        wmax[wave] = mx;
      }
    }
    // (the first half of the workgroup adds up the slabs, the second the chunks before this
    // one in its slab, four loads in flight each: one after the other the up to 30 reads were
    // a third of the kernel's time on short rows)
    static_assert(NT == 2 * BK_BINS, "one thread per bin for the slabs, one for the chunks");
    uint32_t tot = 0, before = 0;
    {
      const uint32_t bin  = tid & (BK_BINS - 1);
      const uint32_t slab = chunk / p.chunks_per_slab;
      if (tid < BK_BINS) {
        for (uint32_t s0 = 0; s0 < p.n_slabs; s0 += 4) {
          uint32_t v[4];
#pragma unroll
          for (uint32_t j = 0; j < 4; ++j)
            v[j] = r.slab_tot[(uint64_t)(s0 + j < p.n_slabs ? s0 + j : s0) * BK_BINS + bin];
#pragma unroll
          for (uint32_t j = 0; j < 4; ++j)
            if (s0 + j < p.n_slabs) {
              tot += v[j];
              if (s0 + j < slab) before += v[j];
            }
        }
      } else {
        uint32_t sum = 0;
        for (uint32_t c0 = slab * p.chunks_per_slab; c0 < chunk; c0 += 4) {
          uint32_t v[4];
#pragma unroll
          for (uint32_t j = 0; j < 4; ++j) v[j] = r.chunk_hist[(uint64_t)(c0 + j < chunk ? c0 + j : c0) * BK_BINS + bin];
#pragma unroll
          for (uint32_t j = 0; j < 4; ++j)
            if (c0 + j < chunk) sum += v[j];
        }
        whist[bin] = sum;  // (whist is free until the first tile)
      }
    }
    const uint32_t incl = wave_incl_scan_u32(tot);
    if (tid < BK_BINS && lane == 63) wave_tot[wave] = incl;
    if (p.flags) {
      // an attempt goes through only if every bin that needs sorting fits the registers of the
      // bin sort: decided from the bins' totals, the same way by every workgroup
      uint32_t longest = (tid < BK_BINS && (tid & 1) == 0) ? tot : 0u;
#pragma unroll
      for (int sft = 32; sft > 0; sft >>= 1) longest = max(longest, (uint32_t)__shfl_xor((int)longest, sft, 64));
      if (tid < BK_BINS && lane == 0) bin_base[wave] = longest;  // (bin_base is free until the first tile)
    }
    __syncthreads();
    if (p.flags) {
      uint32_t longest = 0;
      for (int w = 0; w < BK_BINS / 64; ++w) longest = max(longest, bin_base[w]);
      const bool ok = longest <= p.cap;
      if (chunk == 0 && tid == 0) p.flags[1] = ok ? 1u : 0u;
      if (!ok) return;
      __syncthreads();
    }
    if (tid < BK_BINS) {
      uint32_t start = incl - tot;
      for (int w = 0; w < wave; ++w) start += wave_tot[w];
      gpos[tid] = start + before + whist[tid];
      if (chunk == 0) {
        r.bin_start[tid] = start;
        if (tid == BK_BINS - 1) r.bin_start[BK_BINS] = p.n;
        if (tid == 0) {  // (the wavefronts' results are in place since the barrier above)
          unsigned long long mn = wmin[0], mx = wmax[0];
          for (int w = 1; w < NW; ++w) {
            mn = wmin[w] < mn ? wmin[w] : mn;
            mx = wmax[w] > mx ? wmax[w] : mx;
          }
          r.key_range[0] = mn;
          r.key_range[1] = mx;
        }
      }
    }
    __syncthreads();
  }

  KeyT* kbuf       = r.buf_keys0;
  PayT* pbuf       = r.buf_pay0;
  KeyT* kout       = r.keys_out;
  int64_t* pout    = r.pay_out;
  uint32_t* my_hist = whist + wave * BK_BINS;

  for (uint32_t t = tile0; t < tile_end; ++t) {
    const uint32_t t0    = t * TILE;
    const uint32_t valid = p.n - t0 < (uint32_t)TILE ? p.n - t0 : (uint32_t)TILE;
    uint32_t b[IPT], rk[IPT];
    for (int i = tid; i < NW * BK_BINS; i += NT) whist[i] = 0;
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const KeyT k = KeyOps<KeyT>::to_key(el[i], p.xform);
      if (p.keys_travel) el[i] = k;
      b[i] = bin_of(tab, k);
    }
    lds_barrier();
    // (slots past the end of the row in the last tile hold no key)
#pragma unroll
    for (int i = 0; i < IPT; ++i) rk[i] = wave_rank<9>(my_hist, b[i], wbase + i * 64 < valid, p.rank_by_add);
    lds_barrier();
    uint32_t tot = 0;
    if (tid < BK_BINS) {
#pragma unroll
      for (int w = 0; w < NW; ++w) tot += whist[w * BK_BINS + tid];
    }
    const uint32_t incl = wave_incl_scan_u32(tot);
    if (tid < BK_BINS && lane == 63) wave_tot[wave] = incl;
    lds_barrier();
    if (tid < BK_BINS) {
      uint32_t run = incl - tot;
      for (int w = 0; w < wave; ++w) run += wave_tot[w];
      bin_base[tid] = run;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const uint32_t c            = whist[w * BK_BINS + tid];
        whist[w * BK_BINS + tid] = run;
        run += c;
      }
    }
    lds_barrier();
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      if (wbase + i * 64 < valid) {
        const uint32_t q = my_hist[b[i]] + rk[i];
        skeys[q]         = el[i];
        if constexpr (HAS_PAY) spay[q] = pv[i];
        sbin[q] = (uint16_t)b[i];
      }
    }
    // the next tile is asked for while this one is written out
    if (t + 1 < tile_end) load_tile(t + 1);
    lds_barrier();
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t q = (uint32_t)tid + i * NT;
      if (q < valid) {
        const uint32_t bin = sbin[q];
        const uint32_t dst = gpos[bin] + (q - bin_base[bin]);
        if (p.direct_equal && (bin & 1u)) {
          if (kout) kout[dst] = skeys[q];  // (keys_out is NULL where keys travel)
          if constexpr (PAY == PAY_IDX32) pout[dst] = (int64_t)spay[q] + p.index_offset;
          if constexpr (PAY == PAY_I64) pout[dst] = spay[q];
        } else {
          kbuf[dst] = skeys[q];
          if constexpr (HAS_PAY) pbuf[dst] = spay[q];
        }
      }
    }
    lds_barrier();
    if (tid < BK_BINS) gpos[tid] += tot;
    // (the next tile's first barrier comes before anything reads gpos again)
  }
}

// ---------------------------------------------------------------------------------------
// bin sort
// ---------------------------------------------------------------------------------------
// A bin too long for the registers: LSD passes by this one workgroup between the two scratch
// buffers, a tile of NT * IPT elements at a time.  Per pass one read of the bin counts the
// digit, then the tiles are walked in order: rank within the tile, stage in LDS in
// tile-sorted order, write every digit value's run to its place.  A bin that came out longer
// than the sample promised is sorted this way (at about a third of the speed per element: the
// runs are written in pieces of lines), and so is every bin of a row that a caller sends down
// this path although it is longer than the path is meant for.
template <typename KeyT, int PAY, int IPT>
__device__ __forceinline__ void bucket_sort_long(
  const BucketParams& p,
  const BucketRow<KeyT, typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type>& r, uint32_t start, uint32_t len, KeyT base, int nbits, int xform, uint32_t* whist,
  uint32_t* wave_tot, KeyT* skeys,
  typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type* spay, uint32_t* gbase /* RADIX */,
  uint32_t* tbase /* RADIX */)
{
  constexpr int NT = BK_NT, NW = NT / 64, TILE = NT * IPT;
  constexpr int NG = NT / RADIX, WPG = NW / NG;
  using PayT = typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type;
  constexpr bool HAS_PAY = PAY != PAY_NONE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t wbase = (uint32_t)wave * (64 * IPT) + lane;
  uint32_t* my_hist    = whist + wave * RADIX;
  const uint32_t dv    = tid & (RADIX - 1);
  const int grp        = wave / (RADIX / 64);
  KeyT* kout           = r.keys_out;
  int64_t* pout        = r.pay_out;
  const bool is_float  = xform == XF_FLOAT;
  const KeyT flip      = xform == XF_SIGNED ? (KeyT)((KeyT)1 << (sizeof(KeyT) * 8 - 1)) : (KeyT)0;
  auto key_of = [&](KeyT raw) { return (KeyT)((is_float ? float_to_key(raw) : (KeyT)(raw ^ flip)) - base); };
  const int npass = (nbits + RADIX_BITS - 1) / RADIX_BITS;  // <= 8

  int cur = 0;
  for (int ps = 0; ps < npass; ++ps) {
    const int shift  = ps * RADIX_BITS;
    const bool last  = ps == npass - 1;
    const KeyT* ksrc = (cur ? r.buf_keys1 : r.buf_keys0) + start;
    const PayT* psrc = (cur ? r.buf_pay1 : r.buf_pay0) + start;
    KeyT* kdst       = (cur ? r.buf_keys0 : r.buf_keys1) + start;
    PayT* pdst       = (cur ? r.buf_pay0 : r.buf_pay1) + start;
    // ---- where every digit value starts in the bin: one read of the bin counts this pass's
    // digit, every wavefront in counters of its own (atomics of several wavefronts on the same
    // few words wait for one another), eight loads per thread in flight ----
    for (int i = tid; i < NW * RADIX; i += NT) whist[i] = 0;
    __syncthreads();
    for (uint32_t e0 = 0; e0 < len; e0 += 8 * NT) {
      KeyT raw[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint32_t e = e0 + u * NT + tid;
        raw[u]           = ksrc[e < len ? e : 0u];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (e0 + u * NT + tid < len) atomicAdd(&my_hist[KeyOps<KeyT>::digit(key_of(raw[u]), shift)], 1u);
    }
    __syncthreads();
    {
      uint32_t c = 0;
      if (tid < RADIX) {
#pragma unroll
        for (int w = 0; w < NW; ++w) c += whist[w * RADIX + tid];
      }
      const uint32_t incl = wave_incl_scan_u32(c);
      if (tid < RADIX && lane == 63) wave_tot[wave] = incl;
      __syncthreads();
      if (tid < RADIX) {
        uint32_t s0 = incl - c;
        for (int w = 0; w < wave; ++w) s0 += wave_tot[w];
        gbase[tid] = s0;
      }
      __syncthreads();
    }
    KeyT el[IPT];
    PayT pv[HAS_PAY ? IPT : 1];
    auto load_tile = [&](uint32_t t0) {
      const uint32_t valid = len - t0 < (uint32_t)TILE ? len - t0 : (uint32_t)TILE;
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        const uint32_t e = wbase + i * 64;
        el[i]            = ksrc[t0 + (e < valid ? e : 0u)];
        if constexpr (HAS_PAY) pv[i] = psrc[t0 + (e < valid ? e : 0u)];
      }
    };
    load_tile(0);
    for (uint32_t t0 = 0; t0 < len; t0 += TILE) {
      const uint32_t valid = len - t0 < (uint32_t)TILE ? len - t0 : (uint32_t)TILE;
      for (int i = tid; i < NW * RADIX; i += NT) whist[i] = 0;
      uint32_t d[IPT], rk[IPT];
#pragma unroll
      for (int i = 0; i < IPT; ++i) d[i] = KeyOps<KeyT>::digit(key_of(el[i]), shift);
      lds_barrier();
#pragma unroll
      for (int i = 0; i < IPT; ++i) rk[i] = wave_rank<RADIX_BITS>(my_hist, d[i], wbase + i * 64 < valid, p.rank_by_add);
      lds_barrier();
      uint32_t count = 0, before = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        if (w == grp * WPG) before = count;
        count += whist[w * RADIX + dv];
      }
      const uint32_t incl = wave_incl_scan_u32(count);
      if (lane == 63) wave_tot[wave] = incl;
      lds_barrier();
      {
        uint32_t first = incl - count;
        for (int w = grp * (RADIX / 64); w < wave; ++w) first += wave_tot[w];
        if (grp == 0) tbase[dv] = first;
        uint32_t off   = first + before;
        uint32_t* mine = whist + grp * WPG * RADIX + dv;
#pragma unroll
        for (int w = 0; w < WPG; ++w) {
          const uint32_t c = mine[w * RADIX];
          mine[w * RADIX]  = off;
          off += c;
        }
      }
      lds_barrier();
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        if (wbase + i * 64 < valid) {
          const uint32_t q = my_hist[d[i]] + rk[i];
          skeys[q]         = el[i];
          if constexpr (HAS_PAY) spay[q] = pv[i];
        }
      }
      // the next tile is asked for while this one is written out
      if (t0 + TILE < len) load_tile(t0 + TILE);
      lds_barrier();
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        const uint32_t q = (uint32_t)tid + i * NT;
        if (q < valid) {
          const KeyT raw     = skeys[q];
          const uint32_t dd  = KeyOps<KeyT>::digit(key_of(raw), shift);
          const uint32_t dst = gbase[dd] + (q - tbase[dd]);
          PayT pw{};
          if constexpr (HAS_PAY) pw = spay[q];
          if (last) {
            if (kout) kout[start + dst] = raw;
            if constexpr (PAY == PAY_IDX32) pout[start + dst] = (int64_t)pw + p.index_offset;
            if constexpr (PAY == PAY_I64) pout[start + dst] = pw;
          } else {
            kdst[dst] = raw;
            if constexpr (HAS_PAY) pdst[dst] = pw;
          }
        }
      }
      lds_barrier();
      if (grp == 0) gbase[dv] += count;
      // (three barriers of the next tile come before anything reads gbase or tbase again)
    }
    // What this pass wrote to global memory is read by other threads of this workgroup next:
    // the barrier orders that at workgroup scope (the wavefronts of a workgroup share their
    // CU's vector cache, which the stores went through).
    __syncthreads();
    cur ^= 1;
  }
}

// grid: one workgroup per pair of bins (2g: the keys between two splitters, sorted here;
// 2g + 1: the keys equal to splitter g, which only need copying, and only if the scatter
// could not write them to the outputs itself).
template <typename KeyT, int PAY, int IPT>
__global__ void __launch_bounds__(BK_NT) bucket_sort_kernel(BucketParams p)
{
  constexpr int NT = BK_NT, CAP = NT * IPT;
  using PayT = typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type;
  constexpr bool HAS_PAY = PAY != PAY_NONE;
  // Keys and payload of a bin side by side in LDS where 16 slots per thread of both fit (8 bytes
  // in all); else room for 16384 elements of the wider of the two, which holds keys and
  // payload side by side for bins of up to 8192 elements and one after the other beyond.
  constexpr int PAYB    = HAS_PAY ? (int)sizeof(PayT) : 0;
  constexpr bool SHARE  = HAS_PAY && IPT == 16 && (int)sizeof(KeyT) + PAYB > 8;
  constexpr int WIDER   = (int)sizeof(KeyT) > PAYB ? (int)sizeof(KeyT) : PAYB;
  constexpr int HALF    = NT * (IPT < 8 ? IPT : 8);  // elements the loop through global memory stages
  __shared__ uint32_t whist[(NT / 64) * RADIX];
  __shared__ uint32_t wave_tot[NT / 64];
  __shared__ __attribute__((aligned(16))) unsigned char store[SHARE ? NT * IPT * WIDER : NT * IPT * ((int)sizeof(KeyT) + PAYB)];
  __shared__ uint32_t gbase[RADIX];
  __shared__ uint32_t tbase[RADIX];
  KeyT* const skeys = reinterpret_cast<KeyT*>(store);
  PayT* const spay  = reinterpret_cast<PayT*>(store + (size_t)(SHARE ? HALF : NT * IPT) * sizeof(KeyT));
  static_assert(!SHARE || (size_t)HALF * (sizeof(KeyT) + sizeof(PayT)) <= sizeof(store), "both halves fit");
  if (p.flags && p.flags[1] == 0) return;  // an attempt that did not go through
  const BucketRow<KeyT, PayT> r(p, blockIdx.y);
  const int tid = threadIdx.x;
  const uint32_t g     = blockIdx.x;
  const uint32_t start = r.bin_start[2 * g], mid = r.bin_start[2 * g + 1], end = r.bin_start[2 * g + 2];
  const uint32_t len   = mid - start;
  const KeyT* kbuf     = r.buf_keys0;
  const PayT* pbuf     = r.buf_pay0;
  KeyT* kout           = r.keys_out;
  int64_t* pout        = r.pay_out;
  auto emit = [&](uint32_t dst, KeyT el, PayT pv) {
    if (kout) kout[dst] = el;
    if constexpr (PAY == PAY_IDX32) pout[dst] = (int64_t)pv + p.index_offset;
    if constexpr (PAY == PAY_I64) pout[dst] = pv;
  };
  if (!p.direct_equal) {
    for (uint32_t e = mid + tid; e < end; e += NT) emit(e, kbuf[e], HAS_PAY ? pbuf[HAS_PAY ? e : 0] : PayT{});
  }
  if (len == 0) return;
  // the keys of the bin lie strictly between the splitters lo and hi: sorted by key - lo, which
  // is below hi - lo and so has that many bits at most
  // (the first bin starts at the row's smallest key, and no bin reaches beyond its largest:
  // the last one would else sort every bit up to the largest key there is)
  const KeyT* spl = r.splitters;
  const KeyT kmax = (KeyT)r.key_range[1];
  const KeyT lo   = g > 0 ? spl[g - 1] : (KeyT)r.key_range[0];
  const KeyT hi   = spl[g] < kmax ? spl[g] : kmax;
  const unsigned long long diff = (unsigned long long)(KeyT)(hi - lo);
  const int nbits = diff ? 64 - __builtin_clzll(diff) : 0;
  const int xform = p.keys_travel ? (int)XF_UNSIGNED : p.xform;
  if (len > p.cap) {
    bucket_sort_long<KeyT, PAY, (IPT < 8 ? IPT : 8)>(p, r, start, len, lo, nbits > 0 ? nbits : 1, xform, whist,
                                                     wave_tot, skeys, spay, gbase, tbase);
    return;
  }
  // The bin in registers, in the instantiation for exactly its number of rows per wavefront:
  // the slots of a wider one would stay live through the passes, and at 16 slots of 8 bytes
  // that costs registers the passes need (144 bytes per lane in scratch memory).
  const BlockSortGeom geo = block_sort_geom<NT>(len);
  auto in_registers = [&](auto rows_tag) {
    constexpr int RR = decltype(rows_tag)::value;
    KeyT el[RR];
    PayT pv[HAS_PAY ? RR : 1];
#pragma unroll
    for (int i = 0; i < RR; ++i) {
      const uint32_t e = geo.wbase + i * 64;
      if (e < len) {
        el[i] = kbuf[start + e];
        if constexpr (HAS_PAY) pv[i] = pbuf[start + e];
      }
    }
    constexpr bool SHARED_LDS = SHARE && NT * RR > HALF;
    unsigned long long bits = nbits >= 64 ? ~0ull : (1ull << nbits) - 1;  // key - lo lies below 2^nbits
    int first_bit           = 0;
    if constexpr (sizeof(KeyT) == 8) first_bit = upper_bits_first(bits, bits);
    for (;;) {
      const bool bad = block_radix_sort_rows<KeyT, PayT, HAS_PAY, NT, RR, RR, SHARED_LDS>(
        whist, wave_tot, skeys, SHARED_LDS ? reinterpret_cast<PayT*>(store) : spay, el, pv, len, lo, nbits, xform,
        p.rank_by_add, bits, first_bit);
      if (first_bit == 0 || !__syncthreads_or(bad ? 1 : 0)) break;  // (first_bit is the same in every thread)
      first_bit = 0;
      bits      = ~0ull;
    }
#pragma unroll
    for (int i = 0; i < RR; ++i) {
      const uint32_t e = geo.wbase + i * 64;
      if (e < len) emit(start + e, el[i], HAS_PAY ? pv[HAS_PAY ? i : 0] : PayT{});
    }
  };
  if (geo.R == 1) in_registers(std::integral_constant<int, 1>{});
  else if (geo.R == 2) in_registers(std::integral_constant<int, 2>{});
  else if (geo.R == 4) in_registers(std::integral_constant<int, 4>{});
  else if constexpr (IPT >= 8) {
    if (geo.R == 8) in_registers(std::integral_constant<int, 8>{});
    else if constexpr (IPT >= 16) in_registers(std::integral_constant<int, 16>{});
  }
}

}  // namespace misort
