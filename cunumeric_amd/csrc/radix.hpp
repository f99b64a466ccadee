// Device radix sort for gfx950: least significant digit first, 8-bit digits, two kernels
// per digit.  Replaces the CUB DeviceRadixSort / DeviceSegmentedRadixSort calls of the
// reference (src/cunumeric/sort/cub_sort.cuh:60-71, 81-105, 120-143, 153-182) and, for
// complex keys, the Thrust merge sort (src/cunumeric/sort/thrust_sort.cuh:61-66, 89-94).
//
// A row is cut into chunks of consecutive tiles (a tile = NT*IPT keys).  Per digit:
//   upsweep_kernel    one workgroup per chunk counts the chunk's digit values (reads keys only)
//                     and adds them to the totals of its slab of chunks;
//   downsweep_kernel  one workgroup per chunk: first the exclusive prefix of those counts over
//                     the digit values and over the chunks before its own (where its keys of
//                     each digit value start), then it walks its tiles in order, carrying the
//                     running start of every digit value, so no workgroup ever waits on another.
// Passes after the first whose digit is the same in every key are skipped: the first upsweep
// ORs the keys and their complements, every later kernel works out the rest from those words
// (plan_pass).
// Keys-only sorts of 8-byte elements: every pass but the last also writes the next pass's digit
// of each key as a byte (SIDE), which the next upsweep counts instead of the keys
// (upsweep_digits_kernel).
// Inside a tile of the downsweep:
//   * wave-striped loads (lane l, item i -> wave_base + i*64 + l), so rank order equals
//     index order and the pass is stable; the next tile is requested before the current one
//     is scattered;
//   * digit ranking with 8 wave64 ballots per key (match-any), one LDS atomic per distinct
//     digit value per wave-row;
//   * keys (and payload) are staged through LDS in tile-sorted order so that the global
//     stores of one digit run are contiguous.
// An earlier single-kernel variant chained tiles by decoupled look-back on per-tile status
// words; at ~40 tiles finishing per microsecond against a ~1-2 us round trip of a
// device-scope load, the look-back walk took 1.2 ms of a 2.0 ms pass on this GPU.
// Rows ("segments") are independent: chunks never cross a row.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "keyspec.hpp"
#include <type_traits>

#include "lanes.hpp"

namespace misort {

// ---------------------------------------------------------------------------------------
// small utility kernels
// ---------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) zero_words_kernel(uint32_t* p, size_t n_words)
{
  // n_words is a multiple of 4 and p is 16-byte aligned (the host lays scratch out so).
  uint4* p4       = reinterpret_cast<uint4*>(p);
  const size_t n4 = n_words >> 2;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4;
       i += (size_t)gridDim.x * blockDim.x)
    p4[i] = make_uint4(0, 0, 0, 0);
}

__global__ void store_u64_kernel(unsigned long long* p, unsigned long long v) { *p = v; }

// ---------------------------------------------------------------------------------------
// geometry shared by the kernels of a pass
// ---------------------------------------------------------------------------------------
struct PassParams {
  const void* keys_in;   // FIRST: raw elements; else keys
  void* keys_out;        // LAST: raw elements (may be NULL when a payload is written); else keys
  const uint8_t* digits_in;  // this pass's digit of every key of keys_in, or NULL (upsweep_digits_kernel)
  uint8_t* digits_out;       // downsweep: the NEXT pass's digit of every key written (always with
                             // SIDE, otherwise only where the pass decides that it pays), or NULL
  uint32_t* side_flags;      // [2][n_rows], or NULL: entry [k & 1][row] = 1 where pass k wrote digits_out
                             // for the row (passes that decide it per row)
  uint32_t n_rows;
  int pass, n_passes;        // which pass this is, of how many
  int digit_base;            // pass j runs over digit digit_base + j of the key (0 unless the sort is by
                             // the upper digits only, upperfirst.hpp); shift = 8 * (digit_base + pass)
  // Passes whose digit is the same in every key move nothing and are skipped, decided on the
  // device: the first upsweep ORs all keys and all complemented keys into key_bits_out
  // (KEY_BITS_SLOTS copies of {or lo, or hi, or-of-complement lo, hi}); a bit varies iff it
  // is set in both.  Every later
  // kernel reads the four words (key_bits) and works out for itself which passes are
  // dead, hence which of the two ping-pong buffers holds its input (key_buf / pay_buf; the
  // keys_in .. pay_out above are what they would be with no pass skipped), and which pass is
  // the next live one (whose digit the side-band carries).  NULL: no pass is skipped.
  const unsigned long long* key_bits;
  unsigned long long* key_bits_out;
  void* key_buf[2];
  void* pay_buf[2];
  int early_last;  // > 0: the highest pass that may write the result in place of the pass over the
                   // most significant digit (see plan_pass); the host launches the scatter of
                   // passes 1 .. early_last in both forms
  const void* pay_in;    // PAY_IDX32: u32 (ignored when FIRST); PAY_I64: int64, NULL => positions
  void* pay_out;         // PAY_IDX32: u32, int64 when LAST; PAY_I64: int64
  uint32_t* chunk_hist;             // [rows * chunks_per_row][RADIX] counts of this pass
  unsigned long long* slab_tot;     // [rows][slabs][RADIX] digit counts per slab of chunks: zero
                                    // before the upsweep, which adds its chunk counts to them
  unsigned long long* slab_tot_next;  // the next pass's slab_tot, cleared by the chunk scan (or NULL)
  unsigned long long* special_blk;  // [rows][chunks_per_row * waves][2] {zeros, nans}, or NULL
  unsigned long long* special_row;  // [rows][4] {zeros, nans, negative zeros, negatives}
  uint64_t row_len;
  int64_t index_offset;
  uint32_t tile;  // keys per tile of the downsweep
  uint32_t tiles_per_row;
  uint32_t tiles_per_chunk;
  uint32_t chunks_per_row;
  uint32_t chunks_per_slab;
  uint32_t slabs_per_row;
  int shift;
  int xform;
  int rank_by_add;    // downsweep: rank with returning LDS adds where the chunk's digits allow
  // Non-NULL where the four-launch path (bucket.hpp) was tried on this row first: the word is 1
  // if that path has written the result already, and every kernel of the radix path then
  // returns at once.
  const uint32_t* done_flag;
  // Non-NULL in the kernels of a sort by the upper digits that is tried first: they run only if
  // the word is non-zero (the sample said that it pays).
  const uint32_t* go_flag;
};

// (every kernel of a pass starts with this)
__device__ __forceinline__ bool pass_called_off(const PassParams& p)
{
  return (p.done_flag && *p.done_flag) || (p.go_flag && *p.go_flag == 0);
}

// key_bits holds this many copies of its four words (their OR counts)
constexpr int KEY_BITS_SLOTS = 8;

// What a kernel of pass p.pass works out from key_bits (all of it uniform).
struct PassPlan {
  bool skip;        // this pass moves nothing
  bool is_last;     // this is the last pass that moves anything: it writes the result
  uint32_t parity;  // dead passes before this one, modulo 2: the ping-pong buffers are swapped
  int next_shift;   // digit position of the next live pass
  int prev_live;    // the last live pass before this one
  int const_digit;  // the digit value every key has in this pass, or -1 if the digit varies
};
// Pass 0 transforms the elements into keys and is never skipped.  The pass over the most
// significant digit transforms them back: without early_last it always runs (and skips the
// counting if its digit is constant); with early_last the last pass whose digit varies
// writes the result instead if it is one of passes 1 .. early_last (the host launches the
// scatter kernel of those passes in both forms, and each finds out here whether it is the one
// to run; pass 0 cannot be first and last at once when it sorts in place, and a pass in the
// upper half would save little for one more launch per pass).
__device__ __forceinline__ PassPlan plan_pass(const PassParams& p)
{
  PassPlan r{false, p.pass == p.n_passes - 1, 0u, p.shift + RADIX_BITS, p.pass - 1, -1};
  if (!p.key_bits) return r;
  auto uniform64 = [](unsigned long long v) {  // same in every lane: keep it in scalar registers
    const uint32_t a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return ((unsigned long long)b << 32) | a;
  };
  unsigned long long w[4] = {0, 0, 0, 0};
#pragma unroll
  for (int sl = 0; sl < KEY_BITS_SLOTS; ++sl) {
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] |= p.key_bits[4 * sl + i];
  }
  const unsigned long long lo = uniform64(w[0] & w[2]);
  const unsigned long long hi = uniform64(w[1] & w[3]);
  // Signed integers (at most 8 bytes: the second pair of words is free for them): a digit
  // below the most significant one that only repeats the sign in every key (small values of
  // both signs: 0x00 / 0xFF) needs no pass either, since the pass over the most significant
  // digit, which then runs because the sign varies, puts the signs apart; the words say that
  // of the values with their sign extension taken out.
  const int base          = p.digit_base;             // pass j <-> digit base + j
  const int top_digit     = base + p.n_passes - 1;    // the most significant digit of the key
  const bool by_magnitude = p.xform == XF_SIGNED && top_digit < 8;
  // bit j: no key varies in digit j (or only with the sign).  Worked out once for all digits:
  // choosing between the words digit by digit where they are used made the compiler keep them
  // in scratch memory.
  uint32_t constant_digits = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const bool in_lo = ((lo >> (8 * j)) & 0xFFull) == 0, in_hi = ((hi >> (8 * j)) & 0xFFull) == 0;
    constant_digits |= (uint32_t)((by_magnitude && j < top_digit) ? in_hi : in_lo) << j;
    constant_digits |= (uint32_t)in_hi << (j + 8);  // digits 8 .. 15 of 16-byte keys
  }
  auto constant = [&](int j) { return ((constant_digits >> (j + base)) & 1u) != 0; };  // j: a pass
  // the last pass that runs
  int last = p.n_passes - 1;
  if (p.early_last) {
    while (last > 0 && constant(last)) --last;
    if (last == 0 || last > p.early_last) last = p.n_passes - 1;
  }
  auto dead = [&](int j) { return j > last || (j > 0 && j < last && constant(j)); };
  for (int j = 1; j < p.pass; ++j) r.parity ^= dead(j) ? 1u : 0u;
  r.skip    = dead(p.pass);
  r.is_last = p.pass == last;
  int nx = p.pass + 1;
  while (nx < last && dead(nx)) ++nx;
  r.next_shift = (nx + base) * RADIX_BITS;
  int pv = p.pass - 1;
  while (pv > 0 && dead(pv)) --pv;
  r.prev_live = pv;
  {
    // (a pass that runs over a constant digit is the one over the most significant digit,
    // which the words of the keys themselves describe)
    const unsigned long long ones = uniform64(p.pass + base < 8 ? w[0] : w[1]);
    const int sh = 8 * ((p.pass + base) & 7);
    if (constant(p.pass) && !(by_magnitude && p.pass < p.n_passes - 1))
      r.const_digit = (int)((ones >> sh) & 0xFFull);
  }
  return r;
}
// index of the ping-pong buffer that holds the input of pass p.pass (>= 1)
__device__ __forceinline__ uint32_t input_buffer(const PassParams& p, const PassPlan& pl)
{
  return (uint32_t)((p.pass - 1) & 1) ^ pl.parity;
}


template <typename T>
__device__ __forceinline__ T wave_incl_scan(T v, int lane)
{
#pragma unroll
  for (int s = 1; s < 64; s <<= 1) {
    const T t = __shfl_up(v, s, 64);
    if (lane >= s) v += t;
  }
  return v;
}

// Forces a value to be materialised here: a load that produces it is waited for at this
// point and not at a later first use.
template <typename T>
__device__ __forceinline__ void pin_value(T& v)
{
  if constexpr (sizeof(T) < 4) {
    uint32_t t = v;
    asm volatile("" : "+v"(t));
    v = (T)t;
  } else if constexpr (sizeof(T) <= 8) {
    asm volatile("" : "+v"(v));
  } else {
    asm volatile("" : "+v"(v.lo));
    asm volatile("" : "+v"(v.hi));
  }
}

// A pass without a byte carry writes the digit side-band only if a tile of the row holds at
// most this many digit values on average (random digits: 256, where it costs 0.4 ms per pass
// at 2^28 keys and saves 0.15-0.3 ms in the next upsweep).
static constexpr uint32_t kSidePresentMax = 64;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load and store of the wave, which would serialise the prefetch of the
// next tile and the draining stores of the previous one with the arithmetic in between.
__device__ __forceinline__ void lds_barrier()
{
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---------------------------------------------------------------------------------------
// upsweep over the digit side-band.  A keys-only pass that is not the last also writes, for
// every key it scatters, that key's digit for the NEXT pass as one byte (downsweep_kernel
// with SIDE).  The next pass then counts those bytes instead of reading the keys again:
// 1 byte per key instead of 4 or 8, and no key arithmetic.  Counters as in
// count8_hist_kernel: every digit value has 32 counters, one per lane modulo 32 and in 32
// different LDS banks, shared by the wavefronts of the workgroup, so the lanes of one atomic
// never queue on a bank.
// ---------------------------------------------------------------------------------------
template <int NT>
__device__ __forceinline__ void count_digit_bytes(const PassParams& p, uint32_t* h /* LDS, RADIX * 32 words, zeroed */)
{
  constexpr int COPIES = 32;
  const uint32_t row   = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x % p.chunks_per_row;
  const uint64_t clen  = (uint64_t)p.tiles_per_chunk * p.tile;
  const uint64_t begin = (uint64_t)chunk * clen;
  uint64_t end         = begin + clen;
  if (end > p.row_len) end = p.row_len;
  const uint64_t n    = end > begin ? end - begin : 0;
  const uint8_t* base = p.digits_in + (uint64_t)row * p.row_len + begin;
  uint32_t* my        = h + (threadIdx.x & (COPIES - 1));
  auto count          = [&](uint32_t d) { atomicAdd(&my[d * COPIES], 1u); };

  // bytes before the first 16-byte boundary and after the last one go one per thread
  uint64_t head = (16 - (reinterpret_cast<uintptr_t>(base) & 15)) & 15;
  if (head > n) head = n;
  const uint64_t nvec = (n - head) / 16;
  const uint4* vbase  = reinterpret_cast<const uint4*>(base + head);
  stream_vectors<4>(vbase, nvec, threadIdx.x, (uint32_t)NT, [&](const uint4& r) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      count(w[e] & 0xFFu);
      count((w[e] >> 8) & 0xFFu);
      count((w[e] >> 16) & 0xFFu);
      count(w[e] >> 24);
    }
  });
  const uint64_t tail0 = head + nvec * 16;
  for (uint64_t i = threadIdx.x; i < head + (n - tail0); i += NT) count(base[i < head ? i : tail0 + (i - head)]);
  __syncthreads();
  uint32_t* out = p.chunk_hist + (uint64_t)blockIdx.x * RADIX;
  unsigned long long* slab =
    p.slab_tot + ((uint64_t)row * p.slabs_per_row + chunk / p.chunks_per_slab) * RADIX;
  for (int d = threadIdx.x; d < RADIX; d += NT) {
    uint32_t c = 0;
    for (int i = 0; i < COPIES; ++i) c += h[d * COPIES + ((i + d) & (COPIES - 1))];  // rotated: no bank queue
    out[d] = c;
    if (c) atomicAdd(&slab[d], (unsigned long long)c);
  }
}

template <int NT>
__global__ void __launch_bounds__(NT) upsweep_digits_kernel(PassParams p)
{
  __shared__ __attribute__((aligned(16))) uint32_t h[RADIX * 32];
  if (pass_called_off(p)) return;
  for (int i = threadIdx.x; i < RADIX * 32; i += NT) h[i] = 0;  // (while the plan's words arrive)
  const bool skip = plan_pass(p).skip;
  __syncthreads();
  if (skip) return;
  count_digit_bytes<NT>(p, h);
}

// ---------------------------------------------------------------------------------------
// upsweep: digit counts of one chunk.  Each wave owns one contiguous quarter of the chunk
// and a private LDS histogram.  SPECIALS (first pass of a keys-only float sort) also counts
// zeros / NaNs per wave sub-chunk for the patch that restores their bit patterns.
// ---------------------------------------------------------------------------------------
template <typename KeyT, bool FIRST, bool SPECIALS, int NT>
__global__ void __launch_bounds__(NT) upsweep_kernel(PassParams p)
{
  constexpr int NW = NT / 64;
  // Four counters per digit value and wave, chosen by lane and laid out next to each other
  // (different LDS banks): when a few digit values dominate, lanes that would queue up on
  // one counter are spread over four.
  constexpr int COPIES = 4;
  constexpr int WORDS  = NW * RADIX * COPIES > RADIX * 32 ? NW * RADIX * COPIES : RADIX * 32;
  __shared__ __attribute__((aligned(16))) uint32_t lhist[WORDS];
  __shared__ unsigned long long wg_bits[FIRST ? NW * 4 : 1];
  if (pass_called_off(p)) return;
  const uint32_t row   = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x % p.chunks_per_row;
  // (the counters are cleared while the words of the plan arrive)
  for (int i = threadIdx.x; i < ((!FIRST && !SPECIALS) ? WORDS : NW * RADIX * COPIES); i += NT) lhist[i] = 0;
  if constexpr (!FIRST) {
    const PassPlan plan = plan_pass(p);
    if (plan.skip) return;  // every key has the same digit: the scatter of this pass is skipped too
    if (plan.const_digit >= 0) {
      // a pass that runs over a digit that no key varies in (the pass over the most
      // significant digit where it is not left out): the counts are the lengths of the
      // chunks, no key needs to be read
      const uint64_t clen = (uint64_t)p.tiles_per_chunk * p.tile, b0 = (uint64_t)chunk * clen;
      const uint64_t b1   = b0 + clen < p.row_len ? b0 + clen : p.row_len;
      const uint32_t cnt  = b1 > b0 ? (uint32_t)(b1 - b0) : 0u;
      for (int d = threadIdx.x; d < RADIX; d += NT) {
        const uint32_t c = d == plan.const_digit ? cnt : 0u;
        p.chunk_hist[(uint64_t)blockIdx.x * RADIX + d] = c;
        if (c)
          atomicAdd(&p.slab_tot[((uint64_t)row * p.slabs_per_row + chunk / p.chunks_per_slab) * RADIX + d],
                    (unsigned long long)c);
      }
      return;
    }
    if (p.key_bits) p.keys_in = input_buffer(p, plan) ? p.key_buf[1] : p.key_buf[0];
    if constexpr (!SPECIALS) {
      // the last live pass wrote this pass's digits as bytes for this row: count those
      if (p.digits_in && p.side_flags && p.side_flags[(uint64_t)(plan.prev_live & 1) * p.n_rows + row]) {
        __syncthreads();
        count_digit_bytes<NT>(p, lhist);
        return;
      }
    }
  }
  __syncthreads();

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const KeyT* in        = reinterpret_cast<const KeyT*>(p.keys_in) + (uint64_t)row * p.row_len;
  const uint64_t clen   = (uint64_t)p.tiles_per_chunk * p.tile;
  // Counting zeros and NaNs needs each wavefront on a range of its own (their order is
  // rebuilt from per-wavefront counts); otherwise the wavefronts of the workgroup walk the
  // chunk together, one stream per workgroup.
  constexpr bool SPLIT  = SPECIALS;
  const uint64_t sub    = SPLIT ? clen / NW : clen;
  const uint64_t begin  = (uint64_t)chunk * clen + (SPLIT ? (uint64_t)wave * sub : 0);
  uint64_t end          = begin + sub;
  if (end > p.row_len) end = p.row_len;
  const uint32_t first = SPLIT ? (uint32_t)lane : threadIdx.x;
  const uint32_t width = SPLIT ? 64u : (uint32_t)NT;
  uint32_t* my = lhist + wave * (RADIX * COPIES) + (lane & (COPIES - 1));

  uint32_t n_zero = 0, n_nan = 0, n_negzero = 0, n_neg = 0;
  // FIRST: OR of the keys and of their complements (which bits vary over the whole input)
  unsigned long long or_lo = 0, or_hi = 0, nor_lo = 0, nor_hi = 0;
  // (sw = 1: the words of signed integers are wanted too; decided once, outside the loop: with
  // the test inside it the first upsweep of every other type ran 7 % longer)
  auto count = [&](KeyT raw, auto sw) {
    // (mode 2: the transform is known to be the complex one, so its test leaves the loop too)
    const KeyT k = FIRST ? KeyOps<KeyT>::to_key(raw, decltype(sw)::value == 2 ? (int)XF_COMPLEX : p.xform) : raw;
    if constexpr (FIRST) {
      if constexpr (sizeof(KeyT) == 16) {
        or_lo |= k.lo;
        or_hi |= k.hi;
        nor_lo |= ~k.lo;
        nor_hi |= ~k.hi;
      } else {
        or_lo |= (unsigned long long)k;
        nor_lo |= (unsigned long long)(KeyT)~k;
        if constexpr (decltype(sw)::value == 1) {
          // signed integers: the same for the value with its sign extension taken out
          // (x ^ (x >> all), i.e. x or ~x): bytes that only repeat the sign come out zero
          using S      = typename std::make_signed<KeyT>::type;
          const KeyT x = (KeyT)(k ^ (KeyT)((KeyT)1 << (sizeof(KeyT) * 8 - 1)));
          const KeyT t = (KeyT)(x ^ (KeyT)((S)x >> (sizeof(KeyT) * 8 - 1)));
          or_hi |= (unsigned long long)t;
          nor_hi |= (unsigned long long)(KeyT)~t;
        }
      }
    }
    atomicAdd(&my[KeyOps<KeyT>::digit(k, p.shift) * COPIES], 1u);
  };
  // SPECIALS: zeros, NaNs, negative zeros, and the elements that sort before the zeros
  // (sign set, neither zero nor NaN: counted as sign bits minus the negative zeros and NaNs).
  // Zeros and NaNs are rare, so a whole 16-byte load is asked at once whether it holds any
  // (smallest and largest of the values without their signs), and looked at one by one only then.
  uint32_t n_sign = 0, n_negnan = 0;
  constexpr int KEY_BITS = (int)sizeof(KeyT) * 8;
  auto special_one = [&](KeyT raw) {
    if constexpr (SPECIALS) {
      using F         = FloatBits<KeyT>;
      const bool isn  = float_is_nan(raw);
      const bool isz  = (KeyT)(raw & (KeyT)~F::SIGN) == 0;
      const bool sign = (raw & F::SIGN) != 0;
      n_nan += isn;
      n_zero += isz;
      n_negzero += isz && sign;
      n_negnan += isn && sign;
    }
  };

  // Counting does not care about order, so a lane takes 16 consecutive bytes per load and
  // keeps four loads in flight, issued before the previous four are counted (the LDS
  // atomics of one batch run under the loads of the next); rows that do not start on a
  // 16-byte boundary and the last few keys go one key per lane.
  constexpr int V = sizeof(KeyT) >= 16 ? 1 : 16 / sizeof(KeyT);
  struct alignas(16) Vec {
    KeyT v[V];
  };
  const uint64_t n  = end > begin ? end - begin : 0;
  const KeyT* base  = in + begin;
  auto count_all = [&](auto sw) {
    uint64_t done = 0;
    if (sizeof(Vec) == 16 && (reinterpret_cast<uintptr_t>(base) & 15) == 0) {  // (16-byte keys: one per load)
      constexpr int U     = 4;
      const uint64_t nvec = n / V;
      const Vec* vbase    = reinterpret_cast<const Vec*>(base);
      stream_vectors<U>(vbase, nvec, first, width, [&](const Vec& r) {
#pragma unroll
        for (int e = 0; e < V; ++e) count(r.v[e], sw);
        if constexpr (SPECIALS && sizeof(KeyT) <= 8) {
          using F = FloatBits<KeyT>;
          KeyT least = (KeyT)~(KeyT)0, most = 0;
#pragma unroll
          for (int e = 0; e < V; ++e) {
            const KeyT t = (KeyT)(r.v[e] << 1);  // without the sign
            least        = t < least ? t : least;
            most         = t > most ? t : most;
            n_sign += (uint32_t)(r.v[e] >> (KEY_BITS - 1));
          }
          if (least == 0 || most > (KeyT)(F::EXP << 1)) {
#pragma unroll
            for (int e = 0; e < V; ++e) special_one(r.v[e]);
          }
        }
      });
      done = nvec * V;
    }
    for (uint64_t i = done + first; i < n; i += width) {
      const KeyT raw = base[i];
      count(raw, sw);
      if constexpr (SPECIALS && sizeof(KeyT) <= 8) {
        n_sign += (uint32_t)(raw >> (KEY_BITS - 1));
        special_one(raw);
      }
    }
  };
  if (FIRST && sizeof(KeyT) <= 8 && p.key_bits_out && p.xform == XF_SIGNED)
    count_all(std::integral_constant<int, 1>{});
  else if (FIRST && sizeof(KeyT) == 8 && p.xform == XF_COMPLEX)
    count_all(std::integral_constant<int, 2>{});
  else
    count_all(std::integral_constant<int, 0>{});

  if constexpr (SPECIALS) {
    n_neg = n_sign - n_negzero - n_negnan;
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
      n_zero += __shfl_xor(n_zero, s, 64);
      n_nan += __shfl_xor(n_nan, s, 64);
      n_negzero += __shfl_xor(n_negzero, s, 64);
      n_neg += __shfl_xor(n_neg, s, 64);
    }
    if (lane == 0) {
      const uint64_t e         = ((uint64_t)row * p.chunks_per_row + chunk) * NW + wave;
      p.special_blk[2 * e]     = n_zero;
      p.special_blk[2 * e + 1] = n_nan;
      unsigned long long* ctr  = p.special_row + (uint64_t)row * 4;
      if (n_zero) atomicAdd(&ctr[0], (unsigned long long)n_zero);
      if (n_nan) atomicAdd(&ctr[1], (unsigned long long)n_nan);
      if (n_negzero) atomicAdd(&ctr[2], (unsigned long long)n_negzero);
      if (n_neg) atomicAdd(&ctr[3], (unsigned long long)n_neg);
    }
  }
  if constexpr (FIRST) {
    if (p.key_bits_out) {
#pragma unroll
      for (int s = 32; s > 0; s >>= 1) {
        or_lo |= __shfl_xor(or_lo, s, 64);
        nor_lo |= __shfl_xor(nor_lo, s, 64);
        if (sizeof(KeyT) == 16 || p.xform == XF_SIGNED) {
          or_hi |= __shfl_xor(or_hi, s, 64);
          nor_hi |= __shfl_xor(nor_hi, s, 64);
        }
      }
      if (lane == 0) {
        wg_bits[wave * 4 + 0] = or_lo;
        wg_bits[wave * 4 + 1] = or_hi;
        wg_bits[wave * 4 + 2] = nor_lo;
        wg_bits[wave * 4 + 3] = nor_hi;
      }
    }
  }
  __syncthreads();
  if constexpr (FIRST) {
    // Atomics on one address queue up (about 10 ns each), so a workgroup adds its bits once,
    // to one of KEY_BITS_SLOTS copies of the words, and nobody waits for the result.
    if (p.key_bits_out && threadIdx.x < 4 &&
        (sizeof(KeyT) == 16 || p.xform == XF_SIGNED || (threadIdx.x & 1) == 0)) {
      unsigned long long v = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) v |= wg_bits[w * 4 + threadIdx.x];
      atomicOr(&p.key_bits_out[4 * (blockIdx.x % KEY_BITS_SLOTS) + threadIdx.x], v);
    }
  }
  uint32_t* out = p.chunk_hist + (uint64_t)blockIdx.x * RADIX;
  unsigned long long* slab =
    p.slab_tot + ((uint64_t)row * p.slabs_per_row + chunk / p.chunks_per_slab) * RADIX;
  for (int d = threadIdx.x; d < RADIX; d += NT) {
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const uint4 q = *reinterpret_cast<const uint4*>(&lhist[(w * RADIX + d) * COPIES]);
      c += q.x + q.y + q.z + q.w;
    }
    out[d] = c;
    if (c) atomicAdd(&slab[d], (unsigned long long)c);
  }
}

// ---------------------------------------------------------------------------------------
// downsweep
// ---------------------------------------------------------------------------------------
// Loads one tile (wave-striped) into registers.  Slots past `valid` (partial last tile of
// a row) read slot 0 instead, so that there is one straight-line load sequence; the caller
// replaces them with the all-ones key, which carries the last digit value in every pass
// and ranks after every real key of that value.
template <typename KeyT, int NT, int IPT>
__device__ __forceinline__ void load_tile_keys(const PassParams& p, uint64_t in_base, uint32_t valid,
                                               uint32_t wbase, KeyT (&keys)[IPT])
{
  const KeyT* kin = reinterpret_cast<const KeyT*>(p.keys_in) + in_base;
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const uint32_t o = wbase + i * 64;
    keys[i]          = kin[o < valid ? o : 0u];
  }
}

template <typename PayT, int NT, int IPT>
__device__ __forceinline__ void load_tile_payload(const PassParams& p, uint64_t in_base,
                                                  uint32_t valid, uint32_t wbase, PayT (&pay)[IPT])
{
  const PayT* pin = reinterpret_cast<const PayT*>(p.pay_in) + in_base;
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const uint32_t o = wbase + i * 64;
    pay[i]           = pin[o < valid ? o : 0u];
  }
}

// The scatter writes whole 128-byte lines.  On this GPU a store that covers a full,
// aligned line costs what a linear copy costs, while digit runs of 64 unaligned bytes
// (a 4096-key tile over 256 digit values) made a pass 2.3x slower.  So per digit value
// the workgroup keeps the tail of its run that does not yet fill a line ("carry", fewer
// than G elements) in LDS and writes it together with the next tile's elements of that
// value.  G elements of the narrowest array written are 128 bytes, capped so the carry
// area stays within 64 KB.

//
// SIDE (keys-only passes that are not the last): the pass also writes the digit side-band,
// the NEXT pass's digit of every key as one byte at the key's output position, for
// upsweep_digits_kernel.  A digit run advances by a few dozen bytes of side-band per tile,
// and a 128-byte line written in pieces that L2 evicts one by one costs as much as the
// keys' whole lines, so the bytes have a carry of their own with 128 entries per digit value:
// bytes of positions [brun, run) wait there (brun: start of the first line not yet
// complete), and whenever the run passes a 128-byte boundary the waiting bytes and the new
// ones up to that boundary go out together.
template <typename KeyT, int PAY, bool FIRST, bool LAST, int NT, int IPT, int G, int OCC,
          bool SIDE = false>
__global__ void __launch_bounds__(NT, OCC) downsweep_kernel(PassParams p)
{
  static_assert(!SIDE || (PAY == PAY_NONE && !LAST && (RADIX * G) / NT <= 8),
                "the side-band is written by keys-only passes before the last");
  static_assert(NT % RADIX == 0 && (NT / 64) % (NT / RADIX) == 0, "whole groups of digit owners");
  static_assert((G & (G - 1)) == 0 && (RADIX * G) % NT == 0, "carry slots divide evenly");
  constexpr int NW   = NT / 64;
  constexpr int TILE = NT * IPT;
  using PayT         = typename std::conditional<PAY == PAY_I64, int64_t, uint32_t>::type;
  constexpr int NP   = PAY == PAY_NONE ? 1 : IPT;

  __shared__ uint32_t whist[NW * RADIX];
  // per digit value, for the write-out of the staged tile: global position of staged slot q
  // is dig_base + q; slots below dig_lim are written now; carry slot e goes to old_run + e
  // for e < dig_oldk (0 if the carry is kept)
  __shared__ unsigned long long dig_base[RADIX];
  __shared__ int32_t dig_lim[RADIX];
  __shared__ uint32_t dig_oldk[RADIX];
  __shared__ unsigned long long old_run[RADIX];
  __shared__ uint32_t wave_tot[NW];
  __shared__ __attribute__((aligned(16))) KeyT skeys[TILE];
  __shared__ __attribute__((aligned(16))) PayT spay[PAY == PAY_NONE ? 1 : TILE];
  __shared__ __attribute__((aligned(16))) KeyT ckeys[RADIX * G];
  __shared__ __attribute__((aligned(16))) PayT cpay[PAY == PAY_NONE ? 1 : RADIX * G];
  // side-band: byte carry (slot s of digit value d holds the byte of position brun + s) and,
  // for the write-out of tile n-1, b_pos = brun before the tile and b_tab =
  //   bits 0-7   how many waiting bytes go out (all of them, or 0),
  //   bits 16-23 eb + 128: carried key e goes out directly if e < eb, else into byte-carry
  //              slot e - eb.
  // The same decision for staged slot q rides in dig_lim: (lim << 8) | delta, with q below
  // lim - delta written directly and the rest of the written keys into slot q - (lim - delta).
  constexpr int BL = 128;
  __shared__ __attribute__((aligned(16))) uint8_t bcarry[SIDE ? RADIX * BL : 16];
  __shared__ unsigned long long b_pos[SIDE ? RADIX : 1];
  __shared__ uint32_t b_tab[SIDE ? RADIX : 1];

  if (pass_called_off(p)) return;
  const int tid        = threadIdx.x;
  const int lane       = tid & 63;
  const int wave       = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wbase = wave * (64 * IPT) + lane;

  const uint32_t row      = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk    = blockIdx.x % p.chunks_per_row;
  const uint32_t tile0    = chunk * p.tiles_per_chunk;
  uint32_t tile_end       = tile0 + p.tiles_per_chunk;
  if (tile_end > p.tiles_per_row) tile_end = p.tiles_per_row;
  const uint64_t row_base = (uint64_t)row * p.row_len;
  auto digit_of = [&](KeyT k) { return KeyOps<KeyT>::digit(k, p.shift); };
  int next_shift = p.shift + RADIX_BITS;  // digit position that the side-band carries
  if constexpr (sizeof(KeyT) >= 4) {  // (shorter keys have no middle pass)
    const PassPlan plan = plan_pass(p);
    if (plan.skip) {
      // Every key of the input has the same digit here: the pass would copy every row onto
      // itself, so it moves nothing and the data stays in the buffer it is in (later kernels
      // work that out the same way).  What it owes the next pass remains: zeroed slab totals.
      if (p.slab_tot_next && chunk < p.slabs_per_row && tid < RADIX)
        p.slab_tot_next[((uint64_t)row * p.slabs_per_row + chunk) * RADIX + tid] = 0;
      return;
    }
    // the pass that writes the result is launched in both forms: only the LAST one runs
    if (plan.is_last != LAST) return;
    next_shift = plan.next_shift;
    if (p.key_bits) {
      const bool cur = input_buffer(p, plan) != 0;
      // (The chosen pointers are the same in every lane.  In the kernels with 16 keys per
      // thread, which have no vector register to spare, saying so keeps them in scalar
      // registers; left to the compiler they pushed other values out to scratch memory there.
      // The other kernels were measured slower with it and keep the plain form.)
      auto chosen = [](auto* q) {
        if constexpr (IPT >= 16) {
          const unsigned long long v = (unsigned long long)q;
          const uint32_t a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
          const uint32_t b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
          return (decltype(q))(((unsigned long long)b << 32) | a);
        } else {
          return q;
        }
      };
      if (!FIRST) {
        p.keys_in = chosen(cur ? p.key_buf[1] : p.key_buf[0]);
        p.pay_in  = chosen(cur ? p.pay_buf[1] : p.pay_buf[0]);
      }
      if (!LAST) {
        p.keys_out = chosen(cur ? p.key_buf[0] : p.key_buf[1]);
        p.pay_out  = chosen(cur ? p.pay_buf[0] : p.pay_buf[1]);
      }
    }
  }

  // thread d < RADIX owns digit value d: global position of its next unwritten element
  // and how many elements of it wait in the carry
  unsigned long long run = 0;
  uint32_t carry_n       = 0;
  unsigned long long brun = 0;  // SIDE: first position whose side-band byte is not yet written

  auto tile_valid = [&](uint32_t t) -> uint32_t {
    const uint64_t rem = p.row_len - (uint64_t)t * TILE;
    return rem < (uint64_t)TILE ? (uint32_t)rem : (uint32_t)TILE;
  };

  // Without SIDE (sorts with a payload, 16-byte keys): whether this pass writes the side-band
  // anyway, byte by byte next to the keys.  That costs a partly written 128-byte line per digit
  // value and tile, so it pays only where few digit values are in use (long runs per tile);
  // decided below from the row's counts, the same way by every workgroup of the row.
  constexpr bool ADAPT = !SIDE && !LAST && sizeof(KeyT) >= 4 && (PAY != PAY_NONE || sizeof(KeyT) > 4);
  bool side_on = false;
  KeyT* kout = reinterpret_cast<KeyT*>(p.keys_out);
  auto emit  = [&](unsigned long long dst, KeyT k, PayT v) {
    if (LAST) {
      if (kout) kout[dst] = KeyOps<KeyT>::from_key(k, p.xform);
    } else {
      kout[dst] = k;
      if constexpr (ADAPT) {
        if (side_on) p.digits_out[dst] = (uint8_t)KeyOps<KeyT>::digit(k, next_shift);
      }
    }
    if (PAY == PAY_IDX32) {
      if (LAST)
        reinterpret_cast<int64_t*>(p.pay_out)[dst] = (int64_t)v + p.index_offset;
      else
        reinterpret_cast<uint32_t*>(p.pay_out)[dst] = (uint32_t)v;
    } else if (PAY == PAY_I64) {
      reinterpret_cast<int64_t*>(p.pay_out)[dst] = (int64_t)v;
    }
  };

  uint32_t* my_hist    = whist + wave * RADIX;
  // How a wave ranks its keys, chosen once per workgroup.  The cheap way is one returning LDS
  // add per key on the wave's counter of the key's digit value (1 LDS instruction instead of
  // 41 vector instructions).  It is stable only because the LDS of gfx950 serves those lanes
  // of ONE instruction that hit the same word in ascending lane order.  That order is not in
  // the ISA manual; it is what the hardware does (misort_selftest_lds_lane_order runs 10^9
  // and more lane operations under contention against the ballot match and counts the
  // differences: none), and PassParams::rank_by_add = 0 switches the use of it off.  Each
  // same-word lane costs about 3 LDS clocks, so with a digit value that holds more than an
  // eighth of the chunk (low-entropy digits, runs of equal keys) the ballot match is the
  // faster one: the chunk's counts from the upsweep decide.
  bool rank_by_add = false;
  {
    // ---- where this chunk's keys of every digit value start (the chunk scan) ----
    // Chunks of a row are grouped in slabs whose digit counts the upsweep has added up
    // (slab_tot).  Start of digit value d for this chunk = row start + keys of smaller digit
    // values in the whole row + keys of d in the slabs before this chunk's + keys of d in
    // the chunks before it inside its slab.  Every workgroup works that out for itself:
    // slabs_per_row + at most chunks_per_slab - 1 coalesced 1 KB reads, issued in batches.
    const uint32_t slab      = chunk / p.chunks_per_slab;
    unsigned long long total = 0, before = 0;
    uint32_t mine            = 0;
    if (tid < RADIX) {
      const unsigned long long* st = p.slab_tot + ((uint64_t)row * p.slabs_per_row) * RADIX + tid;
      for (uint32_t sb = 0; sb < p.slabs_per_row; sb += 16) {
        unsigned long long v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = sb + i < p.slabs_per_row ? st[(uint64_t)(sb + i) * RADIX] : 0ull;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (sb + i < slab) before += v[i];
          total += v[i];
        }
      }
      const uint32_t* h = p.chunk_hist + ((uint64_t)row * p.chunks_per_row) * RADIX + tid;
      for (uint32_t cb = slab * p.chunks_per_slab; cb < chunk; cb += 16) {
        uint32_t v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = cb + i < chunk ? h[(uint64_t)(cb + i) * RADIX] : 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) before += v[i];
      }
      mine = h[(uint64_t)chunk * RADIX];
      // the slab totals of the next pass start at zero: the first slabs_per_row chunks of a
      // row clear one slab each (nobody reads that buffer during this pass)
      if (p.slab_tot_next && chunk < p.slabs_per_row)
        p.slab_tot_next[((uint64_t)row * p.slabs_per_row + chunk) * RADIX + tid] = 0;
    }
    // exclusive scan of the row totals over the digit values (threads 0 .. RADIX-1), and the
    // largest and the sum of this chunk's counts; the tables are free before the first step
    const unsigned long long incl = wave_incl_scan(total, lane);
    uint32_t m = mine, c = mine;
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
      m = max(m, (uint32_t)__shfl_xor((int)m, s, 64));
      c += (uint32_t)__shfl_xor((int)c, s, 64);
    }
    // how many digit values a tile of this row holds on average, in 1/65536: a value with
    // count c is in a tile with probability min(1, c * TILE / row_len)
    uint32_t present = 0;
    if (tid < RADIX) {
      const unsigned long long t = total * (unsigned long long)TILE;
      present = t >= p.row_len ? 65536u : (uint32_t)((t << 16) / p.row_len);
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) present += (uint32_t)__shfl_xor((int)present, s, 64);
    if (lane == 63 && wave < RADIX / 64) {
      old_run[wave]  = incl;
      dig_lim[wave]  = (int32_t)m;
      dig_oldk[wave] = c;
      dig_base[wave] = present;
    }
    __syncthreads();
    unsigned long long base = 0;
    uint32_t mx = 0, tot = 0;
    present = 0;
#pragma unroll
    for (int w = 0; w < RADIX / 64; ++w) {
      if (w < wave) base += old_run[w];
      mx = max(mx, (uint32_t)dig_lim[w]);
      tot += dig_oldk[w];
      present += (uint32_t)dig_base[w];
    }
    if constexpr (ADAPT) {
      if (p.digits_out) {
        side_on = __builtin_amdgcn_readfirstlane((int)(present <= kSidePresentMax * 65536u)) != 0;
        if (chunk == 0 && tid == 0 && p.side_flags)
          p.side_flags[(uint64_t)(p.pass & 1) * p.n_rows + row] = side_on ? 1u : 0u;
      }
    }
    if (tid < RADIX) run = row_base + base + incl - total + before;
    brun = run;
    // returning adds unless one digit value holds more than an eighth of the chunk
    if (p.rank_by_add)
      rank_by_add = __builtin_amdgcn_readfirstlane((int)(mx * 8u <= tot)) != 0;
    __syncthreads();
  }
  // The thread index as a value the compiler cannot trace back to threadIdx: LDS addresses
  // formed from it are recomputed where they are used (one or two instructions) instead of
  // being held in registers across the whole tile loop, which the register budget of a
  // 1024-thread workgroup has no room for.
  auto fresh_tid = [&]() -> uint32_t {
    uint32_t t = tid;
    asm volatile("" : "+v"(t));
    return t;
  };
  const bool pay_synth = (PAY == PAY_IDX32) ? FIRST : (PAY == PAY_I64 && p.pay_in == nullptr);

  // One step of the software pipeline.  Tile n sits in the registers ck/cp (requested one
  // step ago).  The step first writes out tile n-1, which the previous step left staged in
  // LDS, then requests tile n+1 into nk/np, and only then ranks and stages tile n: the
  // stores and the loads drain while the wave does the ranking arithmetic (one workgroup
  // owns the CU, so nothing else would overlap them).  The keys of tile n are forced to
  // have arrived before any of that is issued: the hardware counts loads and stores in one
  // in-order counter, so waiting for them later would also wait for everything younger.
  // (The step after the last tile, which only writes out, is a separate instantiation:
  // with one body for both, the compiler's wait-count bookkeeping sees a path that skips
  // the wait for tile n and then waits for it again in the middle of the ranking, behind
  // the requests just issued.)
  auto step = [&](auto drain, KeyT(&ck)[IPT], PayT(&cp)[NP], KeyT(&nk)[IPT], PayT(&np)[NP],
                  uint32_t n) {
    constexpr bool has_cur  = !decltype(drain)::value;
    const bool has_prev     = n > tile0;
    const uint64_t tile_off = (uint64_t)n * TILE;  // within the row
    const uint32_t valid    = has_cur ? tile_valid(n) : 0u;
    const uint32_t pvalid   = has_prev ? tile_valid(n - 1) : 0u;
    const bool more         = n + 1 < tile_end;
    lds_barrier();  // staging and bookkeeping of tile n-1 complete

    if (has_cur) {
#pragma unroll
      for (int i = 0; i < IPT; ++i) pin_value(ck[i]);
      if (PAY != PAY_NONE && !pay_synth) {
#pragma unroll
        for (int i = 0; i < NP; ++i) pin_value(cp[i]);
      }
    }

    uint32_t dfr[SIDE ? 8 : 1];  // SIDE: byte-carry writes of carried keys, held until the barrier
    if (has_prev) {
      // ---- carried elements whose line tile n-1 completes ----
      // thread x = tid + i*NT holds carry slot e = x % G of digit value x / G
      // All LDS reads of a batch are issued before the first store so that they overlap.
      constexpr int NB  = RADIX * G / NT;
      constexpr int BB  = NB < 8 ? NB : 8;
      if constexpr (SIDE) {
        // ---- side-band bytes whose line tile n-1 completes: thread x = tid + i*NT holds
        // the four bytes w = x % 32 of digit value x / 32
        constexpr int ND = RADIX * (BL / 4) / NT;
        const uint32_t ft = fresh_tid();
#pragma unroll
        for (int i = 0; i < ND; ++i) {
          const uint32_t x   = ft + i * NT;
          const uint32_t d   = x / (BL / 4);
          const uint32_t w4  = (x % (BL / 4)) * 4;
          const uint32_t cnt = b_tab[d] & 0xFFu;
          if (w4 < cnt) {
            const uint32_t val           = reinterpret_cast<const uint32_t*>(bcarry)[x];
            const unsigned long long pos = b_pos[d] + w4;
            uint8_t* o                   = p.digits_out + pos;
            if (cnt - w4 >= 4 && (pos & 3) == 0) {
              *reinterpret_cast<uint32_t*>(o) = val;
            } else {
              o[0] = (uint8_t)val;
              if (cnt - w4 > 1) o[1] = (uint8_t)(val >> 8);
              if (cnt - w4 > 2) o[2] = (uint8_t)(val >> 16);
              if (cnt - w4 > 3) o[3] = (uint8_t)(val >> 24);
            }
          }
        }
      }
      const uint32_t bt = fresh_tid();
      const uint32_t e  = bt % G;  // NT is a multiple of G
#pragma unroll 1
      for (int i0 = 0; i0 < NB; i0 += BB) {
        uint32_t ok[BB];
        uint32_t tb[SIDE ? BB : 1];
        unsigned long long orun[BB];
        KeyT bk[BB];
        PayT bv[PAY == PAY_NONE ? 1 : BB];
#pragma unroll
        for (int j = 0; j < BB; ++j) {
          const uint32_t x = bt + (i0 + j) * NT;
          const uint32_t d = x / G;
          ok[j]            = dig_oldk[d];
          if constexpr (SIDE) tb[j] = b_tab[d];
          orun[j]          = old_run[d];
          bk[j]            = ckeys[x];
          if (PAY != PAY_NONE) bv[j] = cpay[x];
        }
#pragma unroll
        for (int j = 0; j < BB; ++j) {
          if constexpr (SIDE) dfr[j] = ~0u;
          if (e < ok[j]) {
            emit(orun[j] + e, bk[j], PAY == PAY_NONE ? PayT{} : bv[PAY == PAY_NONE ? 0 : j]);
            if constexpr (SIDE) {
              const int32_t eb = (int32_t)((tb[j] >> 16) & 0xFFu) - 128;
              const uint32_t b = KeyOps<KeyT>::digit(bk[j], next_shift);
              if ((int32_t)e < eb) {
                p.digits_out[orun[j] + e] = (uint8_t)b;
              } else {
                // into the byte carry, but only after the barrier: its old bytes are being read
                const uint32_t d = (bt + (i0 + j) * NT) / G;
                dfr[j]           = ((d * BL + (uint32_t)((int32_t)e - eb)) << 8) | b;
              }
            }
          }
        }
      }
    }
    for (int i = tid; i < NW * RADIX; i += NT) whist[i] = 0;
    // staged tile n-1 into registers (all LDS reads first, in two dependent rounds); after
    // the barrier only registers, the digit tables and the carry are involved
    const uint32_t at = fresh_tid();
    KeyT ak[IPT];
    PayT av[NP];
    unsigned long long abase[IPT];
    int32_t alim[IPT];
    if (has_prev) {
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        ak[i] = skeys[at + i * NT];
        if (PAY != PAY_NONE) av[i] = spay[at + i * NT];
      }
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        const uint32_t d = digit_of(ak[i]);
        abase[i]         = dig_base[d];
        alim[i]          = dig_lim[d];
      }
    }
    lds_barrier();  // carry and staged tile read; per-wave counters zeroed
    // staged slots of tile n-1, from the registers filled before the barrier: to global
    // memory up to the line boundary of their digit value, the rest into the carry
    auto write_staged = [&]() {
      if constexpr (SIDE) {
        constexpr int NB = RADIX * G / NT;
#pragma unroll
        for (int j = 0; j < NB; ++j)
          if (dfr[j] != ~0u) bcarry[dfr[j] >> 8] = (uint8_t)dfr[j];
      }
#pragma unroll
      for (int i = 0; i < IPT; ++i) {
        const uint32_t q = at + i * NT;
        const PayT v     = PAY == PAY_NONE ? PayT{} : av[PAY == PAY_NONE ? 0 : i];
        const int32_t lim = SIDE ? (alim[i] >> 8) : alim[i];
        if (q < pvalid) {
          if ((int32_t)q < lim) {
            emit(abase[i] + q, ak[i], v);
            if constexpr (SIDE) {
              const int32_t blim = lim - (alim[i] & 0xFF);
              const uint32_t b   = KeyOps<KeyT>::digit(ak[i], next_shift);
              if ((int32_t)q < blim)
                p.digits_out[abase[i] + q] = (uint8_t)b;
              else
                bcarry[digit_of(ak[i]) * BL + (uint32_t)((int32_t)q - blim)] = (uint8_t)b;
            }
          } else {
            const uint32_t d = digit_of(ak[i]);
            const uint32_t c = d * G + (uint32_t)((int32_t)q - lim);
            ckeys[c]         = ak[i];
            if (PAY != PAY_NONE) cpay[c] = v;
          }
        }
      }
    };
    if constexpr (!has_cur) {
      if (has_prev) write_staged();
    }
    if constexpr (has_cur) {
    // Stores before loads: with the requests for tile n+1 issued first, the same stores
    // made a pass a fifth slower.
    if (has_prev) write_staged();
    // keys and payload of tile n+1 are not needed before the next step
    const uint32_t nvalid = more ? tile_valid(n + 1) : 0u;
    if (more) {
      if (PAY != PAY_NONE && !pay_synth)
        load_tile_payload<PayT, NT, NP>(p, row_base + tile_off + TILE, nvalid, wbase, np);
      load_tile_keys<KeyT, NT, IPT>(p, row_base + tile_off + TILE, nvalid, wbase, nk);
    }

#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const KeyT k = FIRST ? KeyOps<KeyT>::to_key(ck[i], p.xform) : ck[i];
      ck[i]        = (wbase + i * 64 < valid) ? k : KeyOps<KeyT>::max_key();
    }
    if (PAY != PAY_NONE && pay_synth) {
      // PAY_IDX32 adds index_offset when widening in the last pass
      const uint64_t pos0 = tile_off + (PAY == PAY_I64 ? (uint64_t)p.index_offset : 0ull);
#pragma unroll
      for (int i = 0; i < IPT; ++i) cp[i] = (PayT)(pos0 + wbase + i * 64);
    }

    // ---- rank tile n within the wave ----
    // match-any: per key the lanes of the wave whose digit equals mine, from 8 ballots; m is
    // the digit bit spread over a word and p & ~(bal ^ m) one three-input bit operation
    // (0xF0 & ~(0xCC ^ 0xAA) = 0x90).  Two keys are matched side by side so the wait states
    // between a compare and the use of its mask are filled with the other key's work.
    uint32_t rank[IPT];
    if (rank_by_add) {
      // One returning LDS add per key: the value returned is the number of keys of this digit
      // value that the wave has seen before this lane (earlier wave-rows, lower lanes of this
      // one), because the LDS of this GPU serves the lanes of one instruction that hit the
      // same word in lane order (see rank_by_add above).
      // A wave-row whose 64 keys hold one or two digit values (runs of equal keys, which the
      // earlier passes have brought together) would queue up on one or two counters, 64 deep
      // in all: there the first lane of each group adds the group's size and the rank is the
      // value it gets plus the number of lower lanes of the group.  Looking for such rows
      // costs more than the add itself, so the first and the last wave-row of the tile are
      // asked first, and the others only if one of the two is such a row.
      struct Groups {
        bool grouped;     // the row holds at most two digit values (same in every lane)
        bool first;       // this lane belongs to the group of lane 0
        uint32_t second;  // first lane of the other group (0 if there is none)
        uint64_t mine;    // the lanes of this lane's group
      };
      auto groups_of = [&](uint32_t d) {
        Groups g;
        const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
        const uint64_t m0 = __ballot(d == d0);
        g.second          = ~m0 ? (uint32_t)__builtin_ctzll(~m0) : 0u;
        const uint32_t d1 = (uint32_t)__builtin_amdgcn_readlane((int)d, (int)g.second);
        const uint64_t m1 = __ballot(d == d1);
        g.grouped         = (m0 | m1) == ~0ull;
        g.first           = d == d0;
        g.mine            = g.first ? m0 : m1;
        return g;
      };
      if (groups_of(digit_of(ck[0])).grouped || groups_of(digit_of(ck[IPT - 1])).grouped) {
#pragma unroll
        for (int i = 0; i < IPT; ++i) {
          const uint32_t d = digit_of(ck[i]);
          const Groups g   = groups_of(d);
          uint32_t r       = 0;
          if (!g.grouped || lane == (g.first ? 0u : g.second))
            r = atomicAdd(&my_hist[d], g.grouped ? (uint32_t)__popcll(g.mine) : 1u);
          if (g.grouped) {
            const uint32_t r0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)r);
            const uint32_t r1 = (uint32_t)__builtin_amdgcn_readlane((int)r, (int)g.second);
            r = (g.first ? r0 : r1) +
                __builtin_amdgcn_mbcnt_hi((uint32_t)(g.mine >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)g.mine, 0u));
          }
          rank[i] = r;
        }
      } else {
#pragma unroll
        for (int i = 0; i < IPT; ++i) rank[i] = atomicAdd(&my_hist[digit_of(ck[i])], 1u);
      }
    } else {
    auto finish_rank = [&](int i, uint32_t d, uint32_t plo, uint32_t phi) {
      const uint32_t below = __builtin_amdgcn_mbcnt_hi(phi, __builtin_amdgcn_mbcnt_lo(plo, 0u));
      const uint32_t cnt   = __popc(plo) + __popc(phi);
      // The lowest peer adds the group's size; LDS executes a wave's operations in order,
      // so the read that follows sees the counter after this wave-row and no later one.
      if (below == 0) atomicAdd(&my_hist[d], cnt);
      const uint32_t delta = cnt - below;
      const uint32_t after =
        __hip_atomic_load(&my_hist[d], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      rank[i] = after - delta;
    };
#pragma unroll
    for (int i = 0; i + 1 < IPT; i += 2) {
      const uint32_t d0 = digit_of(ck[i]);
      const uint32_t d1 = digit_of(ck[i + 1]);
      uint32_t plo0 = ~0u, phi0 = ~0u, plo1 = ~0u, phi1 = ~0u;
#pragma unroll
      for (int b = 0; b < RADIX_BITS; ++b) {
        uint32_t m0 = (uint32_t)((int32_t)(d0 << (31 - b)) >> 31);
        uint32_t m1 = (uint32_t)((int32_t)(d1 << (31 - b)) >> 31);
        asm("" : "+v"(m0));  // compare the spread word itself: one shift less per bit
        asm("" : "+v"(m1));
        const uint64_t bal0 = __ballot(m0 != 0);
        const uint64_t bal1 = __ballot(m1 != 0);
        plo0 = __builtin_amdgcn_bitop3_b32(plo0, (uint32_t)bal0, m0, 0x90);
        phi0 = __builtin_amdgcn_bitop3_b32(phi0, (uint32_t)(bal0 >> 32), m0, 0x90);
        plo1 = __builtin_amdgcn_bitop3_b32(plo1, (uint32_t)bal1, m1, 0x90);
        phi1 = __builtin_amdgcn_bitop3_b32(phi1, (uint32_t)(bal1 >> 32), m1, 0x90);
      }
      finish_rank(i, d0, plo0, phi0);
      finish_rank(i + 1, d1, plo1, phi1);
    }
    if (IPT & 1) {
      const uint32_t d = digit_of(ck[IPT - 1]);
      uint32_t plo = ~0u, phi = ~0u;
#pragma unroll
      for (int b = 0; b < RADIX_BITS; ++b) {
        uint32_t m = (uint32_t)((int32_t)(d << (31 - b)) >> 31);
        asm("" : "+v"(m));
        const uint64_t bal = __ballot(m != 0);
        plo = __builtin_amdgcn_bitop3_b32(plo, (uint32_t)bal, m, 0x90);
        phi = __builtin_amdgcn_bitop3_b32(phi, (uint32_t)(bal >> 32), m, 0x90);
      }
      finish_rank(IPT - 1, d, plo, phi);
    }
    }
    lds_barrier();

    // ---- per-digit tile counts, offsets of each wave, what is written now ----
    // Every thread takes digit value dv = tid % RADIX and the waves of its quarter of the
    // workgroup; all of them read the value's NW per-wave counts.
    constexpr int NG  = NT / RADIX;  // thread groups, each covering all digit values
    constexpr int WPG = NW / NG;     // waves whose counters a group rewrites
    const uint32_t dt = fresh_tid();
    const uint32_t dv = dt & (RADIX - 1);
    const int grp     = wave / (RADIX / 64);  // same for the whole wave
    uint32_t count = 0, before = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == grp * WPG) before = count;  // keys of dv held by the waves of earlier groups
      count += whist[w * RADIX + dv];
    }
    // exclusive scan of the tile's counts over digit values, done by every group for itself
    // (padding keys of a partial tile carry the last digit value and rank last in it: they
    // are staged past `valid` and never written)
    const uint32_t incl = wave_incl_scan_u32(count);
    if (lane == 63) wave_tot[wave] = incl;
    lds_barrier();
    {
      uint32_t base = 0;
      for (int w = grp * (RADIX / 64); w < wave; ++w) base += wave_tot[w];
      const uint32_t tile_start = base + incl - count;  // first staged slot of this value
      if (grp == 0) {
        uint32_t real = count;
        if (dv == RADIX - 1) real -= (uint32_t)TILE - valid;
        // sequence of this value: [carry_n carried elements | real new elements], element 0
        // at global position run.  Write up to the last line boundary inside it
        // (everything at the end of the chunk).
        const uint32_t total        = carry_n + real;
        const unsigned long long hi = (run + total) & ~(unsigned long long)(G - 1);
        const uint32_t flush        = more ? (hi > run ? (uint32_t)(hi - run) : 0u) : total;
        dig_base[dv] = run + carry_n - tile_start;
        const int32_t lim = (int32_t)(flush + tile_start) - (int32_t)carry_n;
        if constexpr (SIDE) {
          // the side-band goes out in whole 128-byte lines up to the new run position
          // (everything at the end of the chunk); bytes of [brun, run) wait in the byte carry
          const unsigned long long new_run = run + flush;
          unsigned long long nb            = more ? (new_run & ~(unsigned long long)(BL - 1)) : new_run;
          if (nb < brun) nb = brun;
          const uint32_t cnt = nb > brun ? (uint32_t)(run - brun) : 0u;
          long long eb       = (long long)nb - (long long)run;  // > -128
          if (eb > 127) eb = 127;
          b_pos[dv]   = brun;
          b_tab[dv]   = cnt | ((uint32_t)(eb + 128) << 16);
          dig_lim[dv] = (int32_t)(((uint32_t)lim << 8) | (uint32_t)(new_run - nb));
          brun        = nb;
        } else {
          dig_lim[dv] = lim;
        }
        dig_oldk[dv] = flush ? carry_n : 0u;
        old_run[dv]  = run;
        run += flush;
        carry_n = total - flush;
      }
      // per-wave counters become the first staged slot of each wave's keys of dv
      uint32_t* mine = whist + grp * WPG * RADIX + dv;
      uint32_t off   = tile_start + before;
#pragma unroll
      for (int w = 0; w < WPG; ++w) {
        const uint32_t c = mine[w * RADIX];
        mine[w * RADIX]  = off;
        off += c;
      }
    }
    lds_barrier();

    // ---- stage tile n through LDS in tile-sorted order ----
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const uint32_t d = digit_of(ck[i]);
      const uint32_t q = my_hist[d] + rank[i];
      skeys[q]         = ck[i];
      if (PAY != PAY_NONE) spay[q] = cp[i];
    }
    }
  };

  KeyT ka[IPT], kb[IPT];
  PayT pa[NP], pb[NP];
  load_tile_keys<KeyT, NT, IPT>(p, row_base + (uint64_t)tile0 * TILE, tile_valid(tile0), wbase, ka);
  if (PAY != PAY_NONE && !pay_synth)
    load_tile_payload<PayT, NT, NP>(p, row_base + (uint64_t)tile0 * TILE, tile_valid(tile0), wbase, pa);
  for (uint32_t n = tile0; n < tile_end; n += 2) {
    step(std::false_type{}, ka, pa, kb, pb, n);
    if (n + 1 >= tile_end) break;
    step(std::false_type{}, kb, pb, ka, pa, n + 1);
  }
  step(std::true_type{}, ka, pa, kb, pb, tile_end);
}

}  // namespace misort
