// Radix select: the key that a full sort would leave at position kth of every row, found
// without sorting.  One pass per key byte, most significant first:
//   select_hist_kernel   counts the current byte of the keys that still match the bytes
//                        fixed so far (one read of the row),
//   select_pick_kernel   finds the byte value whose bucket holds position kth, fixes it,
//                        and clears the counters for the next pass.
// Once the keys that still match are few (at most an eighth of the row, known after a pick),
// the next histogram pass also writes them out side by side ("candidates"), and the passes
// after that read the candidates instead of the row: with uniform keys the last two of four
// passes then read 1/256 of the data.  The state of a row (SEL_ROW / SEL_APPEND / SEL_CAND)
// lives on the device and is advanced by select_pick_kernel.
// After the last byte the pivot key is complete; partition / argpartition then run ONE
// three-way split pass around it (select_split_kernel).  Where the keys of every chunk go
// (those below / equal to / above the pivot) is put together from what the chunks counted
// during the selection (select_cand_counts_kernel, select_chunk_counts_kernel,
// select_chunk_offsets_kernel), so the row is not read once more to count them.  The reference
// sorts completely for partition (cunumeric/deferred.py:3559-3578); NumPy only asks for
// the element at kth to be in its sorted place with nothing larger before it and nothing
// smaller after it.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include "radix.hpp"

namespace misort {

constexpr int SEL_NT = 512;
// where the histogram pass of a row reads its keys, and whether it writes candidates
constexpr uint32_t SEL_ROW = 0, SEL_APPEND = 1, SEL_CAND = 2;

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

// What the kernels of a selection share.  All arrays live in the caller's scratch memory.
template <typename KeyT>
struct SelectParams {
  const KeyT* in;                 // rows of row_len values
  uint64_t row_len, chunk_len;    // chunk geometry: the one of the split pass that follows
  uint32_t chunks_per_row, n_chunks, n_passes;
  int xform;
  KeyT* prefix;                   // per row: the bytes of the kth key found so far
  unsigned long long* kleft;      // per row: position of kth among the keys that match the prefix
  unsigned long long* ghist;      // per row: RADIX counters of the current pass
  uint32_t* pass_hist;            // [pass][chunk][RADIX]: what each chunk counted when it read the row
  uint32_t* state;                // per row: SEL_ROW / SEL_APPEND / SEL_CAND
  uint32_t* cand_from;            // per row: first pass that read the candidates (n_passes: none did)
  KeyT* cand;                     // per row: cand_cap keys (transformed)
  uint32_t* cand_chunk;           // the chunk each candidate came from
  unsigned long long* cand_n;     // per row: candidates written
  uint64_t cand_cap;
  unsigned long long* n_equal;    // per row: keys equal to the kth key (known after the last pick)
  unsigned long long* above_max;  // per row, three words (misort_select only): smallest key above the kth
                                 // key among the candidates, largest key of the row, smallest key above
                                 // the kth key found by the read of the row itself
  uint32_t* cand_less_eq;         // per chunk: candidates below the kth key, and equal to it
  // for the split pass
  uint32_t* chunk_cls;            // [chunk][4]: keys below / equal to / above the kth key (and a pad)
  unsigned long long* chunk_off;  // [chunk][4]: where the chunk's keys of each class go in the output
};

// grid: n_chunks.  Pass `pass` counts byte `shift / 8` of the keys that match the prefix.
// state[row]: SEL_ROW reads the row; SEL_APPEND reads the row and appends the keys that match
// the prefix to the row's candidates; SEL_CAND reads those candidates (they are keys already),
// spread evenly over the row's workgroups.
template <typename KeyT>
__global__ void __launch_bounds__(SEL_NT) select_hist_kernel(SelectParams<KeyT> p, int pass, int shift)
{
  constexpr int NW = SEL_NT / 64, COPIES = 4;
  // Candidates are collected per wavefront and written out a few hundred at a time: the
  // place in the row's candidate area comes from one counter, and atomics on one address
  // queue up, so there must be few of them.
  constexpr uint32_t CB = 4096 / sizeof(KeyT);
  __shared__ __attribute__((aligned(16))) uint32_t h[NW * RADIX * COPIES];
  __shared__ __attribute__((aligned(16))) KeyT cbuf[NW * CB];
  for (int i = threadIdx.x; i < NW * RADIX * COPIES; i += SEL_NT) h[i] = 0;
  __syncthreads();
  const uint32_t row = blockIdx.x / p.chunks_per_row, chunk = blockIdx.x % p.chunks_per_row;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t* my      = h + wave * (RADIX * COPIES) + (lane & (COPIES - 1));
  const KeyT pre    = p.prefix[row];
  const uint32_t st = p.state[row];
  KeyT* my_cand     = p.cand + (uint64_t)row * p.cand_cap;
  const KeyT* base;
  uint64_t b0, b1;
  if (st == SEL_CAND) {
    const uint64_t n_c = p.cand_n[row];
    const uint64_t per = (n_c + p.chunks_per_row - 1) / p.chunks_per_row;
    base = my_cand;
    b0   = (uint64_t)chunk * per;
    b1   = b0 + per < n_c ? b0 + per : n_c;
    if (b0 > b1) b0 = b1;
  } else {
    base = p.in + (uint64_t)row * p.row_len;
    b0   = (uint64_t)chunk * p.chunk_len;
    b1   = b0 + p.chunk_len;
    if (b1 > p.row_len) b1 = p.row_len;
    if (b0 > b1) b0 = b1;
  }
  constexpr int V = sizeof(KeyT) >= 16 ? 1 : 16 / sizeof(KeyT);
  struct alignas(16) Vec {
    KeyT v[V];
  };
  // 16-byte loads a lane keeps in flight (fewer for 1-byte keys, whose 16 counts per load
  // would not fit the registers otherwise)
  constexpr int U = sizeof(KeyT) == 1 ? 2 : 8;
  // (one instance of the loop per state, so that the plain pass carries none of the rest)
  auto scan = [&](auto state_tag) {
    constexpr uint32_t ST = decltype(state_tag)::value;
    KeyT top{};                 // the largest key seen (wanted of pass 0 by misort_select)
    uint32_t n_buf        = 0;  // APPEND: keys in this wavefront's part of cbuf (same in every lane)
    KeyT* wbuf            = cbuf + wave * CB;
    auto flush = [&] {
      unsigned long long at = 0;
      if (lane == 0) at = atomicAdd(&p.cand_n[row], (unsigned long long)n_buf);
      at = __shfl(at, 0, 64);
      for (uint32_t i = lane; i < n_buf; i += 64) {
        my_cand[at + i]                                     = wbuf[i];
        p.cand_chunk[(uint64_t)row * p.cand_cap + at + i] = blockIdx.x;
      }
      n_buf = 0;
    };
    // APPEND calls this with all lanes of the wavefront present; `valid` marks the real keys
    auto count = [&](KeyT raw, bool valid) {
      const KeyT k     = ST == SEL_CAND ? raw : KeyOps<KeyT>::to_key(raw, p.xform);
      const bool match = valid && select_matches(k, pre, shift);
      if (match) atomicAdd(&my[KeyOps<KeyT>::digit(k, shift) * COPIES], 1u);
      if constexpr (ST == SEL_ROW && sizeof(KeyT) <= 8) top = key_lt(top, k) ? k : top;
      if constexpr (ST == SEL_APPEND) {
        const uint64_t m = __ballot(match);
        if (m) {
          if (match) wbuf[n_buf + __popcll(m & ((1ull << lane) - 1))] = k;
          n_buf += __popcll(m);
        }
      }
    };
    // (asked once per 16-byte load: V more keys per lane fit behind what is there)
    auto flush_if_full = [&] {
      if constexpr (ST == SEL_APPEND)
        if (n_buf > CB - 64 * V) flush();
    };
    // 16-byte loads where the row allows it; in whole batches only when appending, so that the
    // rest is done with the wavefronts intact
    uint64_t i0 = b0;
    if (sizeof(Vec) == 16 && (reinterpret_cast<uintptr_t>(base + b0) & 15) == 0) {
      uint64_t nvec = (b1 - b0) / V;
      if (ST == SEL_APPEND) nvec -= nvec % ((uint64_t)SEL_NT * U);
      const Vec* vb = reinterpret_cast<const Vec*>(base + b0);
      if constexpr (sizeof(Vec) == 16) {
        stream_vectors<U>(vb, nvec, threadIdx.x, SEL_NT, [&](const Vec& r) {
#pragma unroll
          for (int e = 0; e < V; ++e) count(r.v[e], true);
          flush_if_full();
        });
      }
      i0 = b0 + nvec * V;
    }
    if constexpr (ST == SEL_APPEND) {
      for (uint64_t i = i0; i < b1; i += SEL_NT) {  // the same number of rounds for every lane
        const bool valid = i + threadIdx.x < b1;
        count(valid ? base[i + threadIdx.x] : KeyT{}, valid);
        flush_if_full();
      }
      if (n_buf) flush();
    } else {
      for (uint64_t i = i0 + threadIdx.x; i < b1; i += SEL_NT) count(base[i], true);
    }
    if constexpr (ST == SEL_ROW && sizeof(KeyT) <= 8) {
      if (p.above_max && pass == 0) {  // (every row is in this state in pass 0)
        unsigned long long hi = 0;
        if constexpr (sizeof(KeyT) <= 8) hi = top;
#pragma unroll
        for (int s = 32; s > 0; s >>= 1) {
          const unsigned long long h2 = __shfl_xor(hi, s, 64);
          hi = h2 > hi ? h2 : hi;
        }
        if (lane == 0 && b1 > b0) atomicMax(&p.above_max[3 * (uint64_t)row + 1], hi);
      }
    }
  };
  if (st == SEL_ROW) scan(std::integral_constant<uint32_t, SEL_ROW>{});
  else if (st == SEL_APPEND) scan(std::integral_constant<uint32_t, SEL_APPEND>{});
  else scan(std::integral_constant<uint32_t, SEL_CAND>{});
  __syncthreads();
  uint32_t* mine = p.pass_hist + ((uint64_t)pass * p.n_chunks + blockIdx.x) * RADIX;
  for (int d = threadIdx.x; d < RADIX; d += SEL_NT) {
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
#pragma unroll
      for (int e = 0; e < COPIES; ++e) c += h[(w * RADIX + d) * COPIES + e];
    }
    if (c) atomicAdd(&p.ghist[(uint64_t)row * RADIX + d], (unsigned long long)c);
    if (st != SEL_CAND) mine[d] = c;
  }
}

// grid: rows, RADIX threads.  Finds the byte value whose keys include position kleft[row].
// Also advances the row's state: a pass that appended is followed by passes over the
// candidates; a row whose chosen bucket fits the candidate area (and that has two more passes
// to go, so that one of them profits) appends in its next pass.
template <typename KeyT>
__global__ void __launch_bounds__(RADIX) select_pick_kernel(SelectParams<KeyT> p, int pass, int shift)
{
  __shared__ unsigned long long wave_tot[RADIX / 64];
  const uint32_t row = blockIdx.x;
  const int d = threadIdx.x, lane = d & 63, wave = d >> 6;
  unsigned long long* g      = p.ghist + (uint64_t)row * RADIX;
  const unsigned long long c = g[d];
  g[d]                       = 0;  // ready for the next pass
  const unsigned long long incl = wave_incl_scan(c, lane);
  if (lane == 63) wave_tot[wave] = incl;
  const unsigned long long k = p.kleft[row];
  __syncthreads();
  unsigned long long before = incl - c;
  for (int w = 0; w < wave; ++w) before += wave_tot[w];
  if (c != 0 && before <= k && k < before + c) {  // exactly one thread
    p.prefix[row]  = select_with_byte(p.prefix[row], (uint32_t)d, shift);
    p.kleft[row]   = k - before;
    p.n_equal[row] = c;  // (what the last pass leaves here is the count of the whole key)
    const uint32_t st = p.state[row];
    if (st == SEL_APPEND) {
      p.state[row]     = SEL_CAND;
      p.cand_from[row] = (uint32_t)pass + 1;
    } else if (st == SEL_ROW && c <= p.cand_cap && shift >= 16) {
      p.state[row] = SEL_APPEND;
    }
  }
}

// grid-stride: prefix <- 0, kleft <- kth, the row is read, no candidates yet
template <typename KeyT>
__global__ void __launch_bounds__(256) select_init_kernel(SelectParams<KeyT> p, uint32_t rows, unsigned long long kth)
{
  for (uint32_t r = blockIdx.x * 256 + threadIdx.x; r < rows; r += gridDim.x * 256) {
    p.prefix[r]    = KeyT{};
    p.kleft[r]     = kth;
    p.state[r]     = SEL_ROW;
    p.cand_from[r] = p.n_passes;
    p.cand_n[r]    = 0;
    if (p.above_max) {
      p.above_max[3 * (uint64_t)r]     = ~0ull;
      p.above_max[3 * (uint64_t)r + 1] = 0;
      p.above_max[3 * (uint64_t)r + 2] = ~0ull;
    }
  }
}

// grid: n_chunks, after the last pick.  Of the candidates of a row that ended up reading
// them, those that share the bytes of the kth key up to the pass that wrote them (the others
// were told apart by that pass's own count) are compared with the kth key, and the chunk
// each came from gets them added to its "below" or "equal" count (cand_less_eq, zero on entry).
template <typename KeyT>
__global__ void __launch_bounds__(SEL_NT) select_cand_counts_kernel(SelectParams<KeyT> p)
{
  const uint32_t row = blockIdx.x / p.chunks_per_row, chunk = blockIdx.x % p.chunks_per_row;
  const uint32_t from = p.cand_from[row];
  if (from >= p.n_passes) return;
  const int lane = threadIdx.x & 63;
  const KeyT kth      = p.prefix[row];
  const int low_shift = (int)sizeof(KeyT) * 8 - 8 * (int)from - 8;  // the first pass over the candidates
  const uint64_t n_c  = p.cand_n[row];
  const uint64_t per  = (n_c + p.chunks_per_row - 1) / p.chunks_per_row;
  uint64_t b0 = (uint64_t)chunk * per, b1 = b0 + per < n_c ? b0 + per : n_c;
  const KeyT* cand    = p.cand + (uint64_t)row * p.cand_cap;
  const uint32_t* src = p.cand_chunk + (uint64_t)row * p.cand_cap;
  for (uint64_t i0 = b0; i0 < b1; i0 += SEL_NT) {  // the same number of rounds for every lane
    const uint64_t i = i0 + threadIdx.x;
    bool less = false, equal = false;
    uint32_t c = 0;
    if (i < b1) {
      const KeyT k = cand[i];
      c            = src[i];
      if (select_matches(k, kth, low_shift)) {
        less  = key_lt(k, kth);
        equal = key_eq(k, kth);
      }
    }
    // candidates of one chunk lie together in runs, so mostly the whole wavefront adds to one chunk
    const uint64_t any = __ballot(less || equal);
    if (any == 0) continue;
    const uint32_t c0 = __shfl(c, __builtin_ctzll(any), 64);
    if (__ballot((less || equal) && c != c0) == 0) {
      const uint32_t nl = __popcll(__ballot(less)), ne = __popcll(__ballot(equal));
      if (lane == 0) {
        if (nl) atomicAdd(&p.cand_less_eq[2 * (uint64_t)c0], nl);
        if (ne) atomicAdd(&p.cand_less_eq[2 * (uint64_t)c0 + 1], ne);
      }
    } else if (less || equal) {
      atomicAdd(&p.cand_less_eq[2 * (uint64_t)c + (equal ? 1 : 0)], 1u);
    }
  }
}

// grid: n_chunks, RADIX threads, after select_cand_counts_kernel.  Puts together, per chunk,
// how many of its keys lie below the kth key, equal it, and lie above, from what the chunk
// counted in the passes that read the row (a key is below if, at the first byte where it
// leaves the kth key, its byte is smaller) and from its candidates; written in the form the
// split pass expects from a counting pass of its own, which therefore does not run.
template <typename KeyT>
__global__ void __launch_bounds__(RADIX) select_chunk_counts_kernel(SelectParams<KeyT> p)
{
  __shared__ unsigned long long wave_tot[RADIX / 64];
  const uint32_t row = blockIdx.x / p.chunks_per_row, chunk = blockIdx.x % p.chunks_per_row;
  const int d = threadIdx.x, lane = d & 63, wave = d >> 6;
  const uint32_t from = p.cand_from[row];
  const KeyT kth      = p.prefix[row];
  unsigned long long below = 0;
  uint32_t equal           = 0;
  for (uint32_t q = 0; q < from; ++q) {
    const int shift   = (int)sizeof(KeyT) * 8 - 8 - 8 * (int)q;
    const uint32_t kb = KeyOps<KeyT>::digit(kth, shift);
    const uint32_t c  = p.pass_hist[((uint64_t)q * p.n_chunks + blockIdx.x) * RADIX + d];
    if ((uint32_t)d < kb) below += c;
    if (q + 1 == p.n_passes && (uint32_t)d == kb) equal = c;  // only one thread
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) {
    below += __shfl_xor(below, s, 64);
    equal += __shfl_xor(equal, s, 64);
  }
  if (lane == 0) wave_tot[wave] = (below << 32) | equal;  // a chunk has fewer than 2^32 keys
  __syncthreads();
  unsigned long long t = 0;
  for (int w = 0; w < RADIX / 64; ++w) t += wave_tot[w];  // (the halves do not carry into each other)
  uint32_t n_below = (uint32_t)(t >> 32), n_equal = (uint32_t)t;
  if (from < p.n_passes) {
    n_below += p.cand_less_eq[2 * (uint64_t)blockIdx.x];
    n_equal = p.cand_less_eq[2 * (uint64_t)blockIdx.x + 1];
  }
  uint64_t b0 = (uint64_t)chunk * p.chunk_len, b1 = b0 + p.chunk_len;
  if (b1 > p.row_len) b1 = p.row_len;
  if (b0 > b1) b0 = b1;
  const uint32_t len = (uint32_t)(b1 - b0);
  if (d < 4) p.chunk_cls[4 * (uint64_t)blockIdx.x + d] = d == 0 ? n_below : d == 1 ? n_equal : d == 2 ? len - n_below - n_equal : 0u;
}

// grid: rows, 256 threads, after select_chunk_counts_kernel.  Where in the output the keys
// of every chunk go: the row's keys below the kth key first, then those equal to it, then
// those above, each class in the order of the chunks (so that equal keys keep their order).
template <typename KeyT>
__global__ void __launch_bounds__(256) select_chunk_offsets_kernel(SelectParams<KeyT> p)
{
  __shared__ unsigned long long wsum[3][4];
  const uint32_t row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t* cls = p.chunk_cls + 4 * (uint64_t)row * p.chunks_per_row;
  unsigned long long* off = p.chunk_off + 4 * (uint64_t)row * p.chunks_per_row;
  // totals of the classes over the row
  unsigned long long t[3] = {0, 0, 0};
  for (uint32_t c = threadIdx.x; c < p.chunks_per_row; c += 256)
    for (int k = 0; k < 3; ++k) t[k] += cls[4 * (uint64_t)c + k];
  for (int k = 0; k < 3; ++k) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) t[k] += __shfl_xor(t[k], s, 64);
    if (lane == 0) wsum[k][wave] = t[k];
  }
  __syncthreads();
  unsigned long long carry[3];
  const unsigned long long n_below = wsum[0][0] + wsum[0][1] + wsum[0][2] + wsum[0][3];
  const unsigned long long n_equal = wsum[1][0] + wsum[1][1] + wsum[1][2] + wsum[1][3];
  carry[0] = (unsigned long long)row * p.row_len;
  carry[1] = carry[0] + n_below;
  carry[2] = carry[1] + n_equal;
  for (uint32_t c0 = 0; c0 < p.chunks_per_row; c0 += 256) {
    const uint32_t c = c0 + threadIdx.x;
    unsigned long long v[3], incl[3];
    __syncthreads();  // wsum is free again
    for (int k = 0; k < 3; ++k) {
      v[k]    = c < p.chunks_per_row ? cls[4 * (uint64_t)c + k] : 0u;
      incl[k] = wave_incl_scan(v[k], lane);
      if (lane == 63) wsum[k][wave] = incl[k];
    }
    __syncthreads();
    for (int k = 0; k < 3; ++k) {
      unsigned long long before = incl[k] - v[k];
      for (int w = 0; w < wave; ++w) before += wsum[k][w];
      if (c < p.chunks_per_row) off[4 * (uint64_t)c + k] = carry[k] + before;
      carry[k] += wsum[k][0] + wsum[k][1] + wsum[k][2] + wsum[k][3];
    }
  }
}

// The split pass of partition / argpartition.  grid: n_chunks, NT threads.  Every workgroup
// walks its chunk in tiles of NT * IPT values; the values of a tile are brought into the
// order below / equal / above in LDS (each class in input order: lane ranks from ballots,
// wavefront offsets from a scan over the counts per load slot and wavefront) and written out
// from there to the three places of the chunk, consecutive threads to consecutive addresses,
// so that lines are written whole except where a class ends within the tile.  What travels is
// the value as it came in (the key only decides the class), or, with POS, its position in the
// row, staged as a 16-bit place within the tile.
template <typename KeyT, bool POS, int NT, int IPT>
__global__ void __launch_bounds__(NT)
select_split_kernel(SelectParams<KeyT> p, KeyT* __restrict__ values_out, int64_t* __restrict__ pos_out,
                    int64_t index_offset)
{
  constexpr int NW = NT / 64, T = NT * IPT;
  static_assert(T <= 65536 && 2 * IPT * NW <= NT && (IPT * NW) % 64 == 0, "tile geometry");
  using StageT = typename std::conditional<POS, uint16_t, KeyT>::type;
  __shared__ __attribute__((aligned(16))) StageT stage[T];
  __shared__ uint32_t cnt[2][IPT * NW];  // per class (below, equal): count per (load slot, wavefront)
  __shared__ uint32_t tot[2];
  const uint32_t row = blockIdx.x / p.chunks_per_row, chunk = blockIdx.x % p.chunks_per_row;
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const KeyT kth     = p.prefix[row];
  uint64_t b0 = (uint64_t)chunk * p.chunk_len, b1 = b0 + p.chunk_len;
  if (b1 > p.row_len) b1 = p.row_len;
  if (b0 > b1) b0 = b1;
  const KeyT* in = p.in + (uint64_t)row * p.row_len;
  unsigned long long g[3];
  for (int k = 0; k < 3; ++k) g[k] = p.chunk_off[4 * (uint64_t)blockIdx.x + k];
  const uint64_t lane_lt = (1ull << lane) - 1;

  for (uint64_t t0 = b0; t0 < b1; t0 += T) {
    const uint32_t valid = b1 - t0 < (uint64_t)T ? (uint32_t)(b1 - t0) : (uint32_t)T;
    KeyT raw[IPT];
    uint32_t cls[IPT];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t e = i * NT + tid;
      raw[i]           = e < valid ? in[t0 + e] : KeyT{};
    }
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t e = i * NT + tid;
      const KeyT k     = KeyOps<KeyT>::to_key(raw[i], p.xform);
      cls[i]           = e >= valid ? 3u : key_lt(k, kth) ? 0u : key_eq(k, kth) ? 1u : 2u;
      const uint64_t m0 = __ballot(cls[i] == 0), m1 = __ballot(cls[i] == 1);
      if (lane == 0) {
        cnt[0][i * NW + wave] = __popcll(m0);
        cnt[1][i * NW + wave] = __popcll(m1);
      }
    }
    __syncthreads();
    // exclusive scan of the counts of each class in the order (load slot, wavefront): the
    // first two wavefronts take a class each, IPT * NW / 64 counts per lane
    if (wave < 2) {
      constexpr int PER = IPT * NW / 64;
      uint32_t v[PER], sum = 0;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        v[j] = cnt[wave][lane * PER + j];
        sum += v[j];
      }
      const uint32_t incl = wave_incl_scan_u32(sum);
      uint32_t run        = incl - sum;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        cnt[wave][lane * PER + j] = run;
        run += v[j];
      }
      if (lane == 63) tot[wave] = incl;
    }
    __syncthreads();
    const uint32_t n0 = tot[0], n1 = tot[1];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t e  = i * NT + tid;
      const uint64_t m0 = __ballot(cls[i] == 0), m1 = __ballot(cls[i] == 1);
      const uint32_t before0 = cnt[0][i * NW + wave] + __popcll(m0 & lane_lt);
      const uint32_t before1 = cnt[1][i * NW + wave] + __popcll(m1 & lane_lt);
      const uint32_t at = cls[i] == 0 ? before0 : cls[i] == 1 ? n0 + before1 : n0 + n1 + (e - before0 - before1);
      if (cls[i] < 3) {
        if constexpr (POS) stage[at] = (uint16_t)e;
        else stage[at] = raw[i];
      }
    }
    __syncthreads();
    const int64_t tile_pos = (int64_t)t0 + index_offset;
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t e = i * NT + tid;
      if (e < valid) {
        const unsigned long long dst = e < n0 ? g[0] + e : e < n0 + n1 ? g[1] + (e - n0) : g[2] + (e - n0 - n1);
        if constexpr (POS) pos_out[dst] = tile_pos + (int64_t)stage[e];
        else values_out[dst] = stage[e];
      }
    }
    g[0] += n0;
    g[1] += n1;
    g[2] += valid - n0 - n1;
  }
}

// grid: n_chunks, after the last pick; keys of at most 8 bytes.  For callers that want the
// key after the kth one instead of a partitioned row: the smallest key above the kth key,
// (all ones where there is none).  Run twice: with CAND over the candidates of the rows that
// have some (the key is nearly always among them; into word 0 of the row's three), then
// without over the rows themselves (into word 2), where the workgroups of a row leave at once
// unless the answer is still open: as many keys equal the kth key as lie at or before kth,
// and the candidates had nothing above it.  The second launch decides that from word 0 alone,
// which only the first launch writes: a word that its own workgroups update could send a
// workgroup that starts late away from a chunk that holds the answer.  (The largest key of the row, the other word, comes from the first histogram pass.)
template <typename KeyT, bool CAND>
__global__ void __launch_bounds__(SEL_NT) select_above_kernel(SelectParams<KeyT> p)
{
  static_assert(sizeof(KeyT) <= 8, "keys of at most 8 bytes");
  __shared__ unsigned long long wmin[SEL_NT / 64];
  const uint32_t row = blockIdx.x / p.chunks_per_row, chunk = blockIdx.x % p.chunks_per_row;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (p.kleft[row] + 1 < p.n_equal[row]) return;  // the key at kth + 1 equals the kth key
  const KeyT kth = p.prefix[row];
  const KeyT* base;
  uint64_t b0, b1;
  if constexpr (CAND) {
    if (p.cand_from[row] >= p.n_passes) return;
    const uint64_t n_c = p.cand_n[row];
    const uint64_t per = (n_c + p.chunks_per_row - 1) / p.chunks_per_row;
    base = p.cand + (uint64_t)row * p.cand_cap;
    b0   = (uint64_t)chunk * per;
    b1   = b0 + per < n_c ? b0 + per : n_c;
  } else {
    // (plain loads of a word that atomics of the launch before wrote: that launch is complete,
    // and this launch writes word 2 only)
    if (p.above_max[3 * (uint64_t)row] != ~0ull) return;
    base = p.in + (uint64_t)row * p.row_len;
    b0   = (uint64_t)chunk * p.chunk_len;
    b1   = b0 + p.chunk_len;
    if (b1 > p.row_len) b1 = p.row_len;
  }
  if (b0 >= b1) return;
  KeyT above = (KeyT)~(KeyT)0;
  auto look = [&](KeyT raw) {
    const KeyT k = CAND ? raw : KeyOps<KeyT>::to_key(raw, p.xform);
    above        = (k > kth && k < above) ? k : above;
  };
  constexpr int V = 16 / sizeof(KeyT);
  struct alignas(16) Vec {
    KeyT v[V];
  };
  uint64_t i0 = b0;
  if ((reinterpret_cast<uintptr_t>(base + b0) & 15) == 0) {
    const uint64_t nvec = (b1 - b0) / V;
    stream_vectors<4>(reinterpret_cast<const Vec*>(base + b0), nvec, threadIdx.x, SEL_NT, [&](const Vec& r) {
#pragma unroll
      for (int e = 0; e < V; ++e) look(r.v[e]);
    });
    i0 = b0 + nvec * V;
  }
  for (uint64_t i = i0 + threadIdx.x; i < b1; i += SEL_NT) look(base[i]);
  // (Nothing found, or only a key that is all ones: the word stays all ones in its full 64
  // bits, whatever the width of the key, which is what the second launch asks for.)
  unsigned long long lo = above == (KeyT)~(KeyT)0 ? ~0ull : (unsigned long long)above;
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) {
    const unsigned long long l2 = __shfl_xor(lo, s, 64);
    lo = l2 < lo ? l2 : lo;
  }
  if (lane == 0) wmin[wave] = lo;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SEL_NT / 64; ++w) lo = wmin[w] < lo ? wmin[w] : lo;
    if (lo != ~0ull) atomicMin(&p.above_max[3 * (uint64_t)row + (CAND ? 0 : 2)], lo);
  }
}

// grid-stride over rows, after the select_above_kernel launches: the kth key, the key at kth + 1
// (the kth key again while more keys equal it than lie at or before kth, else the smallest
// key above it) and the largest key, as values of the element type.  Floating-point values
// come back in the form the keys keep: zeros as +0, every NaN as the default NaN.
template <typename KeyT>
__global__ void __launch_bounds__(256)
select_emit_kernel(SelectParams<KeyT> p, uint32_t rows, KeyT* __restrict__ kth_out, KeyT* __restrict__ next_out,
                   KeyT* __restrict__ max_out)
{
  for (uint32_t r = blockIdx.x * 256 + threadIdx.x; r < rows; r += gridDim.x * 256) {
    const KeyT kth  = p.prefix[r];
    const KeyT top  = (KeyT)p.above_max[3 * (uint64_t)r + 1];
    const unsigned long long a0 = p.above_max[3 * (uint64_t)r], a2 = p.above_max[3 * (uint64_t)r + 2];
    KeyT above      = (KeyT)(a0 < a2 ? a0 : a2);
    if (above > top) above = top;  // nothing above: the row ends at kth (callers do not ask then)
    if (kth_out) kth_out[r] = KeyOps<KeyT>::from_key(kth, p.xform);
    if (next_out) next_out[r] = KeyOps<KeyT>::from_key(p.kleft[r] + 1 < p.n_equal[r] ? kth : above, p.xform);
    if (max_out) max_out[r] = KeyOps<KeyT>::from_key(top, p.xform);
  }
}

}  // namespace misort
