// C ABI of the MI355X local sort: argument checks, plan, scratch layout, kernel launches.
// Entry points are declared in include/misort.h; each replaces a piece of the reference's
// local_sort<CODE> (src/cunumeric/sort/sort.cu:52-85) as cited there.
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/misort.h"
#include "launcher.hpp"
#include "radix.hpp"
#include "rows_api.hpp"
#include "util_kernels.hpp"
#include "count16.hpp"
#include "count8.hpp"
#include "search.hpp"
#include "select.hpp"
#include "unique.hpp"
#include "selftest.hpp"
#include "bucket.hpp"
#include "upperfirst.hpp"

namespace misort {

static_assert(PAY_I64 == 2, "rows_api.hpp spells the caller-payload kind as 2");

thread_local std::string g_last_error;

static constexpr int kMaxDevices = 64;

// Ranking by returning LDS adds (radix.hpp, rank_by_add) leans on the LDS serving the lanes of
// one instruction that hit the same word in ascending lane order, which gfx950 does and no
// manual promises.  So the library decides per GPU, the first time a sort runs there (or in
// misort_init): ballots if the environment says MISORT_RANK_BALLOT=1 (read once), ballots on
// anything that is not gfx950, and otherwise a short probe on a stream of its own (three
// launches of lds_lane_order_probe_kernel, 25 million lane operations with 256, 4 and 1
// distinct words per wavefront, about 0.35 ms) that compares the returning add with the ballot
// match lane by lane: adds only if not one lane disagrees.  The verdict is kept per GPU.
enum RankMode : int { RANK_UNTESTED = 0, RANK_ADD = 1, RANK_BALLOT = 2 };
static std::atomic<int> g_rank_mode[kMaxDevices];
static std::mutex g_probe_mutex;  // the probe's counters are one pair per GPU

static bool rank_ballot_env()
{
  static const bool v = [] {
    const char* e = getenv("MISORT_RANK_BALLOT");
    return e && *e && *e != '0';
  }();
  return v;
}

static int probe_lane_order(int dev)
{
  std::lock_guard<std::mutex> lock(g_probe_mutex);
  int m = g_rank_mode[dev].load(std::memory_order_acquire);
  if (m != RANK_UNTESTED) return m;
  m = RANK_BALLOT;  // whatever goes wrong below: ballots need no such property
  hipDeviceProp_t prop;
  hipStream_t st = nullptr;
  unsigned long long* counts = nullptr;
  if (hipGetDeviceProperties(&prop, dev) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0 &&
      hipGetSymbolAddress(reinterpret_cast<void**>(&counts), HIP_SYMBOL(g_selftest_counts)) == hipSuccess &&
      hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess) {
    hipLaunchKernelGGL(store_u64_kernel, dim3(1), dim3(1), 0, st, counts, 0ull);
    hipLaunchKernelGGL(store_u64_kernel, dim3(1), dim3(1), 0, st, counts + 1, 0ull);
    const uint32_t masks[3] = {0xFFu, 0x03u, 0x00u};
    for (int i = 0; i < 3; ++i)
      hipLaunchKernelGGL(lds_lane_order_probe_kernel, dim3(256), dim3(1024), 0, st, 32u, masks[i],
                         0x2468ACEu + i, counts);
    unsigned long long h[2] = {0, 1};
    hipError_t e = hipMemcpyAsync(h, counts, sizeof h, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e == hipSuccess && hipGetLastError() == hipSuccess && h[0] == 3ull * 256 * 16 * 32 * 64 && h[1] == 0)
      m = RANK_ADD;
  }
  if (st) hipStreamDestroy(st);
  (void)hipGetLastError();
  g_rank_mode[dev].store(m, std::memory_order_release);
  return m;
}

// 1: this GPU ranks with returning adds, 0: with ballots
static int rank_by_add_on_current_device()
{
  if (rank_ballot_env()) return 0;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int m = g_rank_mode[dev].load(std::memory_order_acquire);
  if (m == RANK_UNTESTED) m = probe_lane_order(dev);
  return m == RANK_ADD ? 1 : 0;
}

// The digit side-band of keys-only sorts (radix.hpp, SIDE) is on unless the environment says
// MISORT_SIDE_BAND=0 when the library is first used.
static bool side_band_default()
{
  static const bool v = [] {
    const char* e = getenv("MISORT_SIDE_BAND");
    return !(e && *e == '0');
  }();
  return v;
}

// Passes over a digit that is the same in every key are skipped unless the environment says
// MISORT_SKIP_PASSES=0 when the library is first used.
static bool skip_passes_default()
{
  static const bool v = [] {
    const char* e = getenv("MISORT_SKIP_PASSES");
    return !(e && *e == '0');
  }();
  return v;
}

// From how many bytes of keys on the last pass whose digit varies writes the result (it costs
// one more launch per middle pass): 256 MB, or what MISORT_EARLY_LAST_BYTES said when the
// library was first used, or what the caller of a *_opts entry point says for that call.
static size_t early_last_min_bytes_default()
{
  static const size_t v = [] {
    const char* e = getenv("MISORT_EARLY_LAST_BYTES");
    return (e && *e) ? (size_t)strtoull(e, nullptr, 10) : (size_t)1 << 28;
  }();
  return v;
}

// What the *_opts entry points let a caller choose per call (misort_options in misort.h);
// everything else runs with the defaults.
struct PlanOptions {
  size_t target_chunks = 0;             // 0: the built-in choice
  long long early_last_min_bytes = -1;  // < 0: the default above
  int bucket_path = -1;                 // < 0: the built-in choice; 0: never; > 0: wherever it is able to run
  unsigned bucket_bins = 0;             // 0: the built-in choice; else splitter intervals, 2 .. 256
  unsigned bucket_cap = 0;              // 0: the built-in choice; else the longest bin sorted in registers
  unsigned bucket_oversample = 0;       // 0: the built-in choice; else samples per bin, 1 .. 32
  int low_cardinality = -1;             // long rows try the four-launch path first: < 0: rows of 2^27 elements
                                        // and more, where the sample holds few distinct keys; 0: never;
                                        // 1: the same for every length; 2: with any sample
  int counting_sort = -1;               // one row of 2-byte values: < 0: counted from the built-in length on;
                                        // 0: never; > 0: whenever the row is too long for the row kernels
  int upper_first = -1;                 // 8-byte keys by their upper 40 bits first (upperfirst.hpp): < 0: from
                                        // 2^25 elements on; 0: never; 1: any length; 2: whatever the sample says
};

static int fail(int code, const std::string& msg)
{
  g_last_error = msg;
  return code;
}

enum KernelId : int {
  K_ZERO = 0,
  K_UPSWEEP,
  K_DOWN_FIRST,
  K_DOWN_MIDDLE,
  K_DOWN_LAST,
  K_DOWN_ONLY,
  K_ROWSORT_WAVE,
  K_ROWSORT_BLOCK,
  K_GATHER,
  K_COPY,
  K_TRANSPOSE,
  K_SPECIAL_SCAN,
  K_SPECIAL_COLLECT,
  K_SPECIAL_PATCH,
  K_COUNT16_HIST,
  K_COUNT16_SCAN,
  K_COUNT16_FILL,
  K_SEARCHSORTED,
  K_UNIQUE_COUNT,
  K_UNIQUE_OFFSETS,
  K_UNIQUE_COMPACT,
  K_COUNT8_HIST,
  K_COUNT8_FILL,
  K_SELECT_INIT,
  K_SELECT_HIST,
  K_SELECT_PICK,
  K_SELECT_COUNTS,
  K_SELECT_NEIGHBOURS,
  K_SELECT_EMIT,
  K_SPLIT,
  K_COLSORT,
  K_BUCKET_PLAN,
  K_BUCKET_COUNT,
  K_BUCKET_SCATTER,
  K_BUCKET_SORT,
  K_UF_PLAN,
  K_UF_FIXUP,
  K_NUM
};

static const char* const kKernelNames[K_NUM] = {
  "zero_words",      "upsweep",
  "downsweep_first", "downsweep_middle", "downsweep_last",  "downsweep_only",
  "rowsort_wave",    "rowsort_block",   "gather",           "copy",
  "swap_last",       "special_scan",    "special_collect",  "special_patch",
  "count16_hist",    "count16_scan",    "count16_fill",     "searchsorted",
  "unique_count",    "unique_offsets",  "unique_compact",   "count8_hist",
  "count8_fill",     "select_init",     "select_hist",      "select_pick",
  "select_counts",   "select_above",    "select_emit",    "select_split",
  "colsort_wave",    "bucket_plan",     "bucket_count",     "bucket_scatter",
  "bucket_sort",     "upper_first_plan", "upper_first_fixup"};

// ---------------------------------------------------------------------------------------
// dtype table
// ---------------------------------------------------------------------------------------
struct DtypeInfo {
  int bytes;
  int xform;
};

static bool dtype_info(int dtype, DtypeInfo& d)
{
  switch (dtype) {
    case MISORT_BOOL:
    case MISORT_UINT8: d = {1, XF_UNSIGNED}; return true;
    case MISORT_INT8: d = {1, XF_SIGNED}; return true;
    case MISORT_UINT16: d = {2, XF_UNSIGNED}; return true;
    case MISORT_INT16: d = {2, XF_SIGNED}; return true;
    case MISORT_FLOAT16: d = {2, XF_FLOAT}; return true;
    case MISORT_UINT32: d = {4, XF_UNSIGNED}; return true;
    case MISORT_INT32: d = {4, XF_SIGNED}; return true;
    case MISORT_FLOAT32: d = {4, XF_FLOAT}; return true;
    case MISORT_UINT64: d = {8, XF_UNSIGNED}; return true;
    case MISORT_INT64: d = {8, XF_SIGNED}; return true;
    case MISORT_FLOAT64: d = {8, XF_FLOAT}; return true;
    case MISORT_COMPLEX64: d = {8, XF_COMPLEX}; return true;
    case MISORT_COMPLEX128: d = {16, XF_COMPLEX}; return true;
    default: return false;
  }
}

// ---------------------------------------------------------------------------------------
// plan
// ---------------------------------------------------------------------------------------
enum Strategy : int { S_EMPTY = 0, S_ROW_WAVE, S_ROW_BLOCK, S_RADIX, S_COUNT16, S_COUNT8, S_BUCKET };

// Tile shape of the downsweep per key width and payload kind: threads, keys per thread,
// elements per 128-byte output line kept in the carry (G), workgroups per CU.  One
// workgroup of 1024 threads fills a CU: staging + carry take most of its 160 KB of LDS.
constexpr int kTileThreads = 1024;
constexpr int kTileOcc     = 1;
constexpr int pay_bytes_of(int pay) { return pay == PAY_NONE ? 0 : (pay == PAY_IDX32 ? 4 : 8); }
constexpr int carry_group(int kb, int pay)
{
  // elements per 128 bytes of the narrowest array written, halved until 256 digit values
  // of carry fit in 64 KB
  const int pb      = pay_bytes_of(pay);
  const int narrow  = (pb != 0 && pb < kb) ? pb : kb;
  int g             = 128 / narrow;
  while (256 * g * (kb + pb) > 64 * 1024) g /= 2;
  return g;
}
constexpr int items_per_thread(int kb, int pay, int nt)
{
  // staging + carry + per-wave counters + bookkeeping within 160 KB
  const int pb     = pay_bytes_of(pay);
  const int budget = 160 * 1024 / kTileOcc - 256 * carry_group(kb, pay) * (kb + pb) -
                     (nt / 64) * 1024 - 6 * 1024;
  int ipt          = budget / (nt * (kb + pb));
  // two key buffers (current and next tile) + payload + ranks stay in registers
  const int cap = kb <= 4 ? (pb == 8 ? 6 : (pb == 0 ? 16 : 8))
                          : (kb == 8 ? (pb == 8 ? 4 : (pb == 0 ? 8 : 7)) : (pb == 8 ? 3 : 4));
  if (ipt > cap) ipt = cap;
  if (ipt < 1) ipt = 1;
  return ipt;
}
template <int KEYBYTES, int PAY>
struct TileCfg {
  static constexpr int NT  = kTileThreads;
  static constexpr int G   = carry_group(KEYBYTES, PAY);
  static constexpr int IPT = items_per_thread(KEYBYTES, PAY, NT);
  static constexpr int OCC = kTileOcc;
  static_assert(IPT >= 1, "tile does not fit");
};

static int tile_size(int key_bytes, int pay)
{
#define MISORT_TILE_CASE(KB)                                                        \
  case KB:                                                                          \
    return pay == PAY_NONE    ? TileCfg<KB, PAY_NONE>::NT * TileCfg<KB, PAY_NONE>::IPT   \
           : pay == PAY_IDX32 ? TileCfg<KB, PAY_IDX32>::NT * TileCfg<KB, PAY_IDX32>::IPT \
                              : TileCfg<KB, PAY_I64>::NT * TileCfg<KB, PAY_I64>::IPT;
  switch (key_bytes) {
    MISORT_TILE_CASE(1)
    MISORT_TILE_CASE(2)
    MISORT_TILE_CASE(4)
    MISORT_TILE_CASE(8)
    default: MISORT_TILE_CASE(16)
  }
#undef MISORT_TILE_CASE
}

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct Plan {
  int strategy = S_EMPTY;
  DtypeInfo dt{};
  size_t volume = 0, row_len = 0, rows = 0;
  bool argsort = false, has_indices_in = false;
  bool gather_values = false;  // complex keys-only: argsort, then gather the elements
  // complex64 keys-only on the radix path: the elements travel through the passes as an 8-byte
  // payload instead (4 bytes more per key and pass than a position, but no gather at the end:
  // 2^26 elements 5.46 -> 4.92 ms)
  bool values_as_payload = false;
  int pay = PAY_NONE;
  int n_passes = 0;
  int tile = 0;
  // radix: a row is cut into chunks of tiles, chunks into slabs for the scan
  size_t tiles_per_row = 0, tiles_per_chunk = 0, chunks_per_row = 0, n_chunks = 0;
  size_t chunks_per_slab = 0, slabs_per_row = 0;
  bool specials = false;  // float keys-only: patch original zero / NaN bit patterns back
  // scratch layout (byte offsets)
  size_t off_special_ctr = 0, special_ctr_bytes = 0;
  size_t off_chunk_hist = 0, off_slab_tot = 0, slab_tot_bytes = 0;
  size_t zero_bytes = 0;  // from off_special_ctr on: what one launch clears before the first pass
  size_t off_keys[2] = {0, 0}, off_pay[2] = {0, 0};
  size_t off_special_blk = 0;
  // digit side-band of keys-only sorts: one byte per key, written by every pass but the last
  // and counted by the next pass's upsweep in place of the keys
  bool side_band = false;
  // the other radix sorts of 4-byte and wider keys: a pass writes the side-band, without the
  // byte carry, only where few digit values are in use; it says so per row in side_flag
  bool side_adaptive = false;
  size_t off_digits = 0, off_side_flag = 0;
  // passes after the first whose digit is the same in every key are skipped (decided on the device from
  // the OR of the keys and of their complements, which the first upsweep leaves in key_bits)
  bool skip_dead_passes = false;
  // > 0: the last pass whose digit varies writes the result if it is one of passes 1 .. this
  // (large sorts only)
  int early_last = 0;
  size_t off_key_bits = 0;
  size_t off_gather_idx = 0, off_gather_src = 0;
  // counting sort of 2-byte keys: chunks of the histogram kernel, counters, their scan
  size_t c16_chunks = 0, c16_chunk_len = 0, off_c16_hist = 0, off_c16_prefix = 0;
  // sample -> count -> scatter -> sort the bins (bucket.hpp): geometry and scratch
  uint32_t bk_split = 0, bk_cap = 0, bk_tile = 0, bk_tiles_per_chunk = 0, bk_chunks = 0, bk_slabs = 0;
  uint32_t bk_oversample = BK_OVERSAMPLE;
  size_t off_bk_splitters = 0, off_bk_slab_tot = 0, off_bk_chunk_hist = 0, off_bk_bin_start = 0;
  size_t off_bk_chunk_range = 0, off_bk_key_range = 0;
  // radix plans of one long row: the four-launch path is tried first, and goes through where
  // the keys take few distinct values (1: if the sample says so; 2: tried with any sample)
  int low_card = 0;
  size_t off_bk_flags = 0;
  // radix plans of 8-byte keys: sorted by the upper five digits first (1: if the sample agrees;
  // 2: whatever it says), the lower three only if the fix-up finds runs too long to sort
  int upper_first = 0;
  size_t off_uf_flags = 0, off_uf_keys = 0;
  size_t total = 0;
};

// Slots per thread of the bin sort (1024 threads): the bin is staged in LDS between the
// passes, 128 KB of it; keys and payload of more than 8 bytes together share that room (side
// by side up to 8192 elements, one after the other beyond).
constexpr int bucket_sort_ipt(int, int) { return 16; }
// The scatter walks tiles of 1024 * 4 elements while that gives every CU a chunk of at most two
// tiles, and tiles as large as the staging area in LDS allows (element, payload, 2 bytes for the
// bin) beyond that.
constexpr int kBucketScatterIptSmall = 4;
// chunks (workgroups) of the count and scatter kernels at most: one per CU for the medium
// rows the path is built for (2^21 int32: 75 us with 256 chunks, 78 with 512); four per CU
// where it is tried on long rows, so that two workgroups of the count kernel are resident per
// CU and cover each other's waits (count of 2^28 int64: 0.69 -> 0.55 ms)
constexpr size_t kBucketMaxChunks = 256, kBucketMaxChunksLong = 1024;
constexpr int bucket_scatter_ipt_large(int kb, int pay)
{
  return kb + pay_bytes_of(pay) <= 4 ? 16 : (kb + pay_bytes_of(pay) <= 12 ? 8 : 4);
}

// Number of chunks a row-set is cut into.  Two per CU measured best from 2^24 to 2^28 keys:
// long chunks keep the downsweep's pipeline and its carried partial lines busy (with one
// tile per chunk every digit run starts and ends on a partial line), and the per-chunk
// bookkeeping (one 256-entry count row, one start row) stays far below the key traffic.
static constexpr size_t kTargetChunks  = 512;
static constexpr size_t kChunksPerSlab = 16;
static constexpr int kUpsweepThreads   = 256;
static constexpr int kUpsweepDigitThreads = 256;  // upsweep over the digit side-band
// values-only sorts of one row of 2-byte elements: counted instead of radix-sorted from this
// length on (two radix passes are ahead below: uniform int16 at 2^24 120 us against 195, level
// near 2^25.5; float16, whose radix sort also restores -0 and NaN payloads, 148 against 111 at
// 2^24, level near 2^23.5)
static constexpr size_t kCount16MinLenInt   = (size_t)1 << 26;
static constexpr size_t kCount16MinLenFloat = (size_t)1 << 24;
static constexpr size_t kCount16Chunks = 512;

// target_chunks: chunks (workgroups) a radix pass over the whole array is cut into; 0 = the
// built-in choice.  It is part of the plan, so the scratch query and the sort must agree on it.
static int make_plan(int dtype, size_t volume, size_t sort_dim_size, bool argsort,
                     bool has_indices_in, Plan& pl, const PlanOptions& opt = PlanOptions{})
{
  const size_t target_chunks = opt.target_chunks;
  if (!dtype_info(dtype, pl.dt)) return fail(MISORT_ERR_DTYPE, "unknown dtype code");
  pl.volume         = volume;
  pl.argsort        = argsort;
  pl.has_indices_in = has_indices_in;
  if (volume == 0) {
    pl.strategy = S_EMPTY;
    return MISORT_OK;
  }
  if (sort_dim_size == 0 || volume % sort_dim_size != 0)
    return fail(MISORT_ERR_SHAPE, "volume is not a multiple of sort_dim_size");
  pl.row_len = sort_dim_size;
  pl.rows    = volume / sort_dim_size;
  if (pl.rows > 0x7FFFFFFFull) return fail(MISORT_ERR_UNSUPPORTED, "more than 2^31-1 rows");

  const bool is_complex = pl.dt.xform == XF_COMPLEX;
  if (!argsort && is_complex) {
    // the composite complex key is not invertible: sort (key, position) and gather
    pl.gather_values = true;
  }
  if (argsort || pl.gather_values) {
    if (has_indices_in || pl.row_len > 0xFFFFFFFFull)
      pl.pay = PAY_I64;
    else
      pl.pay = PAY_IDX32;
  } else {
    pl.pay = PAY_NONE;
  }
  pl.specials = (!argsort && pl.dt.xform == XF_FLOAT);

  if (rowsort_supported(pl.dt.bytes, pl.row_len, pl.pay, pl.gather_values) && pl.rows >= 1 &&
      pl.row_len <= rowsort_wave_max(pl.dt.bytes)) {
    pl.strategy = S_ROW_WAVE;
  } else if (rowsort_supported(pl.dt.bytes, pl.row_len, pl.pay, pl.gather_values) &&
             pl.row_len <= rowsort_block_max(pl.dt.bytes, pl.pay)) {
    pl.strategy = S_ROW_BLOCK;
  } else if (pl.dt.bytes == 2 && pl.pay == PAY_NONE && pl.rows == 1 && opt.counting_sort != 0 &&
             (opt.counting_sort > 0 ||
              pl.row_len >= (pl.dt.xform == XF_FLOAT ? kCount16MinLenFloat : kCount16MinLenInt))) {
    pl.strategy = S_COUNT16;
  } else if (pl.dt.bytes == 1 && pl.pay == PAY_NONE && pl.rows == 1) {
    pl.strategy = S_COUNT8;  // any single row too long for the row kernels
  } else {
    pl.strategy = S_RADIX;
  }
  if (pl.strategy == S_RADIX && pl.gather_values && pl.dt.bytes == 8) {
    pl.gather_values     = false;
    pl.values_as_payload = true;
    pl.pay               = PAY_I64;
    pl.argsort           = true;
    pl.has_indices_in    = true;
  }

  if (pl.strategy == S_RADIX && pl.rows <= 65535 && pl.dt.bytes <= 8 && !pl.gather_values && opt.bucket_path != 0 &&
      (opt.target_chunks == 0 || opt.bucket_path > 0)) {  // (a chunk count is a request to the radix path)
    // Rows of up to about two million elements: four launches in all instead of two per digit.
    const size_t cap_full = (size_t)BK_NT * bucket_sort_ipt(pl.dt.bytes, pl.pay);
    const size_t cap      = opt.bucket_cap ? std::min<size_t>(opt.bucket_cap, cap_full) : cap_full;
    // Up to 256 bins of half of what the registers hold on average: with 16 samples per bin a
    // bin twice the average is a one-in-a-thousand event, and such a bin is still sorted, by the
    // slower loop through global memory.  Where the path ends is measured against the radix
    // passes (random keys, back to back): 4-byte keys are ahead up to 2^21 elements in one row
    // (72 us against 92; 131 against 99 at 3 x 2^20), 8-byte keys as far as the bins fit (108
    // against 202 at 2^21), 2-byte keys, which take two radix passes only, up to 2^19 alone
    // (37 against 40; float16, whose radix sort patches zeros and NaNs afterwards, 2^20) and 2^18
    // with positions, 1-byte keys nowhere (one radix pass: 17-20 us against 21-41).  Several rows
    // side by side while all of them together stay within a length of the same kind: the bin
    // sort is built for latency, one workgroup of 1024 threads per CU and bin, and beyond one or
    // two rounds of bins over the CUs the radix passes move more keys per second (8 rows of
    // int32 at 2^21 in all: 98 against 93; 8-byte keys ahead up to 2^22: 211 against 264 alone,
    // 224 against 329 with positions).
    const bool forced = opt.bucket_path > 0;
    size_t max_len = 128 * cap_full, max_vol = 128 * cap_full;
    if (pl.dt.bytes == 8) max_vol = (size_t)1 << 22;
    if (pl.dt.bytes == 4) max_vol = 96 * cap_full;
    if (pl.dt.bytes == 2)
      max_len = max_vol = (pl.pay != PAY_NONE ? 16 : pl.dt.xform == XF_FLOAT ? 64 : 32) * cap_full;
    if (pl.dt.bytes == 1) max_len = max_vol = 0;
    if (pl.rows == 1) max_vol = max_len;
    if (forced) max_len = max_vol = (size_t)0xFFFFFFFFu / 2;
    if (pl.row_len <= max_len && pl.volume <= max_vol && cap >= 64) {
      size_t bins = opt.bucket_bins ? opt.bucket_bins : (pl.row_len + 1023) / 1024;
      if (bins < 2) bins = 2;
      if (bins > 256) bins = 256;
      pl.strategy = S_BUCKET;
      pl.bk_split = (uint32_t)bins - 1;
      pl.bk_cap   = (uint32_t)cap;
      // 16 samples per bin: a bin of twice the average is a 7e-4 event per bin, one of three
      // times 1e-8.  Rows whose bins average more than 5/12 of the capacity (2.4 times the
      // average fills a bin: 1.5e-5) draw 32 (twice the average: 4e-6), or one sort in six at the
      // longest rows would find a bin that takes the loop through global memory; that costs the
      // plan kernel 8 us more.
      if (pl.row_len > bins * (cap * 5 / 12)) pl.bk_oversample = BK_OVERSAMPLE_MAX;
      if (opt.bucket_oversample >= 1 && opt.bucket_oversample <= (unsigned)BK_OVERSAMPLE_MAX)
        pl.bk_oversample = opt.bucket_oversample;
    }
  }

  size_t off = 0;
  auto take  = [&](size_t bytes) {
    const size_t o = off;
    off += align_up(bytes, 256);
    return o;
  };

  // chunks of the count and scatter kernels of the four-launch path, and its tables
  auto bucket_tables = [&](size_t max_chunks) {
    pl.bk_tile            = BK_NT * (pl.row_len <= ((size_t)1 << 21) ? kBucketScatterIptSmall
                                                                       : bucket_scatter_ipt_large(pl.dt.bytes, pl.pay));
    const size_t tiles    = (pl.row_len + pl.bk_tile - 1) / pl.bk_tile;
    const size_t want     = tiles < max_chunks ? tiles : max_chunks;
    pl.bk_tiles_per_chunk = (uint32_t)((tiles + want - 1) / want);
    pl.bk_chunks          = (uint32_t)((tiles + pl.bk_tiles_per_chunk - 1) / pl.bk_tiles_per_chunk);
    pl.bk_slabs           = (uint32_t)((pl.bk_chunks + kChunksPerSlab - 1) / kChunksPerSlab);
    pl.off_bk_splitters   = take(pl.rows * BK_SLOTS * 8);
    pl.off_bk_slab_tot    = take(pl.rows * pl.bk_slabs * BK_BINS * sizeof(uint32_t));
    pl.off_bk_chunk_hist  = take(pl.rows * pl.bk_chunks * BK_BINS * sizeof(uint32_t));
    pl.off_bk_bin_start   = take(pl.rows * (BK_BINS + 1) * sizeof(uint32_t));
    pl.off_bk_chunk_range = take(pl.rows * pl.bk_chunks * 2 * sizeof(unsigned long long));
    pl.off_bk_key_range   = take(pl.rows * 2 * sizeof(unsigned long long));
    pl.off_bk_flags       = take(2 * sizeof(uint32_t));
  };

  if (pl.strategy == S_BUCKET) {
    bucket_tables(kBucketMaxChunks);
    for (int b = 0; b < 2; ++b) pl.off_keys[b] = take(pl.volume * pl.dt.bytes);
    if (pl.pay != PAY_NONE)
      for (int b = 0; b < 2; ++b) pl.off_pay[b] = take(pl.volume * (pl.pay == PAY_IDX32 ? 4 : 8));
  } else if (pl.strategy == S_RADIX) {
    pl.n_passes      = pl.dt.bytes;  // 8-bit digits
    pl.tile          = tile_size(pl.dt.bytes, pl.pay);
    pl.tiles_per_row = (pl.row_len + pl.tile - 1) / pl.tile;
    size_t target = target_chunks;
    if (target == 0) {
      // two workgroups per CU, which balances the end of a long pass (2^28 keys: 1-3 % faster
      // than one); one per CU below 32 tiles per workgroup at two, where paying a workgroup's
      // start-up once per CU counts for more (2^24 (key, position) pairs 7 % faster with one,
      // 2^25 4 %, 2^26 3 %; level at 32 tiles)
      target = kTargetChunks;
      if (pl.rows * pl.tiles_per_row < 32 * target) target /= 2;
    }
    size_t want = (target + pl.rows - 1) / pl.rows;  // chunks per row aimed at
    if (want < 1) want = 1;
    if (want > pl.tiles_per_row) want = pl.tiles_per_row;
    pl.tiles_per_chunk = (pl.tiles_per_row + want - 1) / want;
    // a chunk's counts are 32-bit words (and the scatter multiplies the largest by 8): at most
    // 2^29 keys per chunk, whatever the caller asked for
    const size_t max_tpc = ((size_t)1 << 29) / (size_t)pl.tile;
    if (pl.tiles_per_chunk > max_tpc) pl.tiles_per_chunk = max_tpc;
    pl.chunks_per_row  = (pl.tiles_per_row + pl.tiles_per_chunk - 1) / pl.tiles_per_chunk;
    pl.n_chunks        = pl.rows * pl.chunks_per_row;
    pl.chunks_per_slab = kChunksPerSlab;
    pl.slabs_per_row   = (pl.chunks_per_row + pl.chunks_per_slab - 1) / pl.chunks_per_slab;
    if (pl.n_chunks > 0x7FFFFFFFull || pl.rows * pl.slabs_per_row > 0x7FFFFFFFull ||
        pl.tiles_per_row > 0xFFFFFFFFull)
      return fail(MISORT_ERR_UNSUPPORTED, "too many chunks for one launch");

    // [special counters | slab totals of even passes | of odd passes]: cleared by one launch
    pl.special_ctr_bytes = pl.specials ? pl.rows * 4 * sizeof(unsigned long long) : 0;
    pl.off_special_ctr   = take(pl.special_ctr_bytes);
    pl.slab_tot_bytes    = pl.rows * pl.slabs_per_row * RADIX * sizeof(unsigned long long);
    pl.off_slab_tot      = take(pl.slab_tot_bytes);
    take(pl.slab_tot_bytes);
    pl.off_side_flag     = take(2 * pl.rows * sizeof(uint32_t));  // per pass parity and row
    pl.off_key_bits      = take(KEY_BITS_SLOTS * 4 * sizeof(unsigned long long));
    pl.zero_bytes        = off - pl.off_special_ctr;
    pl.off_chunk_hist    = take(pl.n_chunks * RADIX * sizeof(uint32_t));

    int n_bufs = pl.n_passes - 1 < 2 ? pl.n_passes - 1 : 2;
    if (n_bufs < 1) n_bufs = 1;  // single-pass sorts stage through one buffer when in == out
    if (pl.specials && n_bufs < 2) n_bufs = 2;  // second buffer collects the special elements
    for (int b = 0; b < n_bufs; ++b) pl.off_keys[b] = take(pl.volume * pl.dt.bytes);
    if (n_bufs == 1) pl.off_keys[1] = pl.off_keys[0];
    if (pl.pay != PAY_NONE) {
      const size_t pb = pl.pay == PAY_IDX32 ? 4 : 8;
      int n_pbufs     = pl.n_passes - 1 < 2 ? pl.n_passes - 1 : 2;
      if (n_pbufs < 1) n_pbufs = 1;
      for (int b = 0; b < n_pbufs; ++b) pl.off_pay[b] = take(pl.volume * pb);
      if (n_pbufs == 1) pl.off_pay[1] = pl.off_pay[0];
    }
    // (8-byte keys: the upsweep saves 7 of 8 bytes per key; with 4-byte keys the extra
    // stores of the scatter cost more than the upsweep saves)
    // (not for keys-only float sorts: the patch of their zeros and NaNs counts on which of the
    // two buffers the last pass leaves free)
    pl.skip_dead_passes = skip_passes_default() && pl.n_passes >= 3 && !pl.specials;
    // (one more launch per middle pass, about 5 us each: from 256 MB of keys on; integers
    // only: the most significant byte of a float key holds the sign and the top of the
    // exponent, which vary in all but contrived inputs)
    pl.early_last =
      (pl.skip_dead_passes && (pl.dt.xform == XF_SIGNED || pl.dt.xform == XF_UNSIGNED) &&
       pl.volume * pl.dt.bytes >= (opt.early_last_min_bytes >= 0 ? (size_t)opt.early_last_min_bytes
                                                                       : early_last_min_bytes_default()))
        ? (int)pl.n_passes / 2
        : 0;
    pl.side_band = side_band_default() && pl.pay == PAY_NONE && pl.n_passes >= 2 && pl.dt.bytes == 8;
    pl.side_adaptive = side_band_default() && !pl.side_band && pl.n_passes >= 2 && pl.dt.bytes >= 4 &&
                       (pl.pay != PAY_NONE || pl.dt.bytes > 4);
    if (pl.side_band || pl.side_adaptive) pl.off_digits = take(pl.volume);
    if (pl.specials)
      pl.off_special_blk =
        take(pl.n_chunks * (kUpsweepThreads / 64) * 2 * sizeof(unsigned long long));
    if (pl.gather_values) {
      pl.off_gather_idx = take(pl.volume * sizeof(int64_t));
      pl.off_gather_src = take(pl.volume * pl.dt.bytes);  // copy of the input when in == out
    }
    // One long row of 4- or 8-byte keys: the four-launch path is tried first (its plan kernel
    // alone, 15 us, where the sample holds more than 255 distinct keys).  With few distinct
    // values every one of them is a splitter with a bin of equal keys behind it, which the
    // scatter fills in input order at the elements' final places: one read to count, one read
    // and one write to place, against a read and a write per key byte.  It shares the radix
    // path's two key and payload buffers.  (Not for keys-only float sorts, whose zeros and NaNs
    // the radix path patches with kernels of its own, and not in place: the scatter writes
    // results while other workgroups still read the input.)
    // (By itself from 2^27 elements on: the plan kernel and the three launches that return at
    // once cost 35-50 us, which is 1 % of a sort of 2^28 keys and 14 % of one of 2^24.)
    if (opt.low_cardinality != 0 && (opt.low_cardinality > 0 || pl.row_len >= ((size_t)1 << 27)) && pl.rows == 1 &&
        (pl.dt.bytes == 4 || pl.dt.bytes == 8) && pl.n_passes >= 3 && !pl.gather_values && !pl.specials &&
        pl.row_len < 0xFFFFFFFFull) {
      pl.low_card = opt.low_cardinality == 2 ? 2 : 1;
      pl.bk_split = BK_SLOTS - 1;
      pl.bk_cap   = (uint32_t)(BK_NT * bucket_sort_ipt(pl.dt.bytes, pl.pay));
      bucket_tables(kBucketMaxChunksLong);
    }
    // Long sorts of 8-byte keys: by the upper five digits first, the lower three only if the
    // fix-up meets runs too long to sort (upperfirst.hpp): five passes and a read of the
    // result instead of eight passes.  From 2^25 elements on, where the 17 launches of the
    // eight-pass sort that return at once (0.1 ms) are a few per cent of what is saved; not in
    // place (the eight-pass sort needs the input again), which the launch sequence checks.
    if (pl.dt.bytes == 8 && pl.n_passes == 8 && !pl.gather_values && opt.upper_first != 0 &&
        opt.target_chunks == 0 && (opt.upper_first > 0 || pl.volume >= ((size_t)1 << 25))) {
      pl.upper_first  = opt.upper_first == 2 ? 2 : 1;
      pl.off_uf_flags = take(2 * sizeof(uint32_t));
      if (pl.pay != PAY_NONE) pl.off_uf_keys = take(pl.volume * pl.dt.bytes);  // the result's keys, for the fix-up
    }
  } else if (pl.strategy == S_COUNT16) {
    // one histogram workgroup per CU and half of the key range, a few rounds of them
    constexpr size_t gran = (size_t)(C16_HIST_NT / 64) * 64 * 8;  // whole 16-byte loads per wavefront
    // at least 2^16 elements per chunk: a workgroup clears and flushes 32768 counters
    size_t want = pl.row_len >> 16;
    if (want < 1) want = 1;
    if (want > kCount16Chunks) want = kCount16Chunks;
    size_t clen           = (pl.row_len + want - 1) / want;
    clen                  = align_up(clen, gran);
    pl.c16_chunk_len      = clen;
    pl.c16_chunks         = (pl.row_len + clen - 1) / clen;
    // per-row special counters and the key counters are cleared by one launch
    pl.special_ctr_bytes = 4 * sizeof(unsigned long long);
    pl.off_special_ctr   = take(pl.special_ctr_bytes);
    pl.off_c16_hist      = take((size_t)C16_BINS * sizeof(unsigned long long));
    pl.off_c16_prefix    = take((size_t)(C16_BINS + 1) * sizeof(unsigned long long));
    if (pl.specials) {
      pl.off_special_blk = take(pl.c16_chunks * (C16_HIST_NT / 64) * 2 * sizeof(unsigned long long));
      pl.off_keys[0]     = take(pl.volume * pl.dt.bytes);  // zeros / NaNs in input order
    }
  } else if (pl.strategy == S_COUNT8) {
    pl.off_c16_hist = take(256 * sizeof(unsigned long long));
  } else {
    // row kernels read a whole row into registers / LDS before writing: no scratch
    take(256);
  }
  pl.total = off;
  return MISORT_OK;
}

// ---------------------------------------------------------------------------------------
// radix launch sequence
// ---------------------------------------------------------------------------------------
struct SortArgs {
  const void* values_in;
  void* values_out;
  const int64_t* indices_in;
  int64_t* indices_out;
  int64_t index_offset;
  char* scratch;
};

template <typename KeyT>
constexpr bool is_float_width()
{
  return std::is_same<KeyT, uint16_t>::value || std::is_same<KeyT, uint32_t>::value ||
         std::is_same<KeyT, uint64_t>::value;
}

// the scatter kernel of one pass
template <typename KeyT, int PAY>
static void launch_downsweep(Launcher& L, const Plan& pl, int id, bool first, bool last,
                             const PassParams& pp)
{
  const dim3 grid((unsigned)pl.n_chunks);
  constexpr int NT  = TileCfg<sizeof(KeyT), PAY>::NT;
  constexpr int IPT = TileCfg<sizeof(KeyT), PAY>::IPT;
  constexpr int OCC = TileCfg<sizeof(KeyT), PAY>::OCC;
  constexpr int G   = TileCfg<sizeof(KeyT), PAY>::G;
  L.run(id, [&] {
    if constexpr (PAY == PAY_NONE && sizeof(KeyT) == 8) {
      if (pp.digits_out) {  // keys-only pass that also writes the digit side-band
        if (first)
          hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, true, false, NT, IPT, G, OCC, true>), grid,
                             dim3(NT), 0, L.stream, pp);
        else
          hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, false, false, NT, IPT, G, OCC, true>), grid,
                             dim3(NT), 0, L.stream, pp);
        return;
      }
    }
    if (first && last)
      hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, true, true, NT, IPT, G, OCC>), grid, dim3(NT), 0,
                         L.stream, pp);
    else if (first)
      hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, true, false, NT, IPT, G, OCC>), grid, dim3(NT),
                         0, L.stream, pp);
    else if (last)
      hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, false, true, NT, IPT, G, OCC>), grid, dim3(NT),
                         0, L.stream, pp);
    else
      hipLaunchKernelGGL((downsweep_kernel<KeyT, PAY, false, false, NT, IPT, G, OCC>), grid, dim3(NT),
                         0, L.stream, pp);
  });
}

template <typename KeyT, int PAY>
static void launch_pass(Launcher& L, const Plan& pl, bool first, bool last, const PassParams& pp)
{
  constexpr int UNT = kUpsweepThreads;
  const dim3 grid((unsigned)pl.n_chunks);

  L.run(K_UPSWEEP, [&] {
    if (pp.digits_in && !pp.side_flags) {  // the last live pass always writes the side-band
      hipLaunchKernelGGL((upsweep_digits_kernel<kUpsweepDigitThreads>), grid, dim3(kUpsweepDigitThreads), 0,
                         L.stream, pp);
      return;
    }
    if (first) {
      if constexpr (is_float_width<KeyT>()) {
        if (pl.specials) {
          hipLaunchKernelGGL((upsweep_kernel<KeyT, true, true, UNT>), grid, dim3(UNT), 0, L.stream, pp);
          return;
        }
      }
      hipLaunchKernelGGL((upsweep_kernel<KeyT, true, false, UNT>), grid, dim3(UNT), 0, L.stream, pp);
    } else {
      hipLaunchKernelGGL((upsweep_kernel<KeyT, false, false, UNT>), grid, dim3(UNT), 0, L.stream, pp);
    }
  });

  const int id = first ? (last ? K_DOWN_ONLY : K_DOWN_FIRST) : (last ? K_DOWN_LAST : K_DOWN_MIDDLE);
  launch_downsweep<KeyT, PAY>(L, pl, id, first, last, pp);
}

static void launch_zero(Launcher& L, void* p, size_t bytes)
{
  const size_t words = align_up(bytes, 16) / 4;
  size_t blocks      = (words / 4 + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks == 0) blocks = 1;
  L.run(K_ZERO, [&] {
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)blocks), dim3(256), 0, L.stream,
                       reinterpret_cast<uint32_t*>(p), words);
  });
}

template <typename KeyT, int PAY>
static void bucket_sort_row(Launcher& L, const Plan& pl, const SortArgs& a, int attempt = 0);

// What distinguishes the runs of the pass sequence below: the plain sort (digit_base 0, all
// digits), and the sort by the upper digits that upperfirst.hpp tries first.
struct RadixRun {
  int digit_base            = 0;        // the first pass's digit
  const uint32_t* done_flag = nullptr;  // the kernels return at once if the word is set
  const uint32_t* go_flag   = nullptr;  // ... or if this one is clear
  void* keys_for_fixup      = nullptr;  // where the last pass puts the keys if the caller wants none
  bool upper_first          = false;
};

template <typename KeyT, int PAY>
static void radix_sort_passes(Launcher& L, const Plan& plan, const SortArgs& a, const RadixRun& run);

template <typename KeyT, int PAY>
static void radix_sort_rows(Launcher& L, const Plan& plan, const SortArgs& a)
{
  char* S = a.scratch;
  // few distinct keys: the four-launch path writes the result, and the kernels below return at once
  const uint32_t* done_flag = nullptr;
  const bool outputs_apart  = (a.values_out == nullptr || a.values_out != a.values_in) &&
                             (a.indices_out == nullptr || a.indices_out != a.indices_in);
  if constexpr (sizeof(KeyT) == 4 || sizeof(KeyT) == 8) {
    if (plan.low_card && outputs_apart) {
      bucket_sort_row<KeyT, PAY>(L, plan, a, plan.low_card);
      done_flag = reinterpret_cast<const uint32_t*>(S + plan.off_bk_flags) + 1;
    }
  }
  if constexpr (sizeof(KeyT) == 8) {
    if (plan.upper_first && outputs_apart) {
      uint32_t* flags = reinterpret_cast<uint32_t*>(S + plan.off_uf_flags);
      UpperFirstParams up{};
      up.keys_in     = a.values_in;
      up.volume      = plan.volume;
      up.row_len     = plan.row_len;
      up.xform       = plan.dt.xform;
      up.low_bits    = RADIX_BITS * upper_first_digit0(plan.dt.xform, plan.row_len);
      up.mode        = plan.upper_first;
      up.rank_by_add = rank_by_add_on_current_device();
      up.flags       = flags;
      up.prior_done  = done_flag;
      L.run(K_UF_PLAN, [&] {
        hipLaunchKernelGGL((upper_first_plan_kernel<KeyT>), dim3(1), dim3(UF_PLAN_NT), 0, L.stream, up);
      });
      RadixRun first;
      first.digit_base  = upper_first_digit0(plan.dt.xform, plan.row_len);
      first.go_flag     = flags;
      first.upper_first = true;
      const bool caller_keys = !plan.argsort || a.values_out != nullptr;
      if (PAY != PAY_NONE && !caller_keys) first.keys_for_fixup = S + plan.off_uf_keys;
      radix_sort_passes<KeyT, PAY>(L, plan, a, first);
      done_flag = flags + 1;
    }
  }
  RadixRun all;
  all.done_flag = done_flag;
  radix_sort_passes<KeyT, PAY>(L, plan, a, all);
}

template <typename KeyT, int PAY>
static void radix_sort_passes(Launcher& L, const Plan& plan, const SortArgs& a, const RadixRun& run)
{
  const size_t eb    = sizeof(KeyT);
  const char* vin    = reinterpret_cast<const char*>(a.values_in);
  char* vout         = reinterpret_cast<char*>(a.values_out);
  // Keys-only float sorts restore the bit patterns of their zeros and NaNs afterwards.  In
  // place, those are set aside before the last pass overwrites the input, in the ping-pong
  // buffer that pass leaves free, which is known on the host only if every pass runs.  Out
  // of place the input outlives the sort, they are taken from there at the end, and passes
  // may be skipped as in every other sort.
  Plan pl                  = plan;
  if (run.upper_first) {
    pl.n_passes -= run.digit_base;
    pl.early_last = 0;  // (the pass over the most significant digit writes the result)
  }
  const bool specials_late = pl.specials && vin != vout;
  if (specials_late && skip_passes_default() && pl.n_passes >= 3) {
    pl.skip_dead_passes = true;
  }
  const int64_t* iin = a.indices_in;
  int64_t* iout      = a.indices_out;
  char* S            = a.scratch;

  unsigned long long* special_row =
    reinterpret_cast<unsigned long long*>(S + pl.off_special_ctr);
  unsigned long long* special_blk =
    reinterpret_cast<unsigned long long*>(S + pl.off_special_blk);

  launch_zero(L, S + pl.off_special_ctr, pl.zero_bytes);

  const size_t pay_bytes     = PAY == PAY_IDX32 ? 4 : 8;
  const bool write_keys_last = !pl.argsort || a.values_out != nullptr;
  // A single pass cannot scatter into the buffer it reads: stage, then copy.
  const bool single     = pl.n_passes == 1;
  const bool alias_keys = single && write_keys_last && !pl.gather_values && vin == vout;
  const bool alias_pay  = single && PAY == PAY_I64 && iin != nullptr && iin == iout;

  PassParams pp{};
  pp.chunk_hist      = reinterpret_cast<uint32_t*>(S + pl.off_chunk_hist);
  pp.special_blk     = pl.specials ? special_blk : nullptr;
  pp.special_row     = special_row;
  pp.row_len         = pl.row_len;
  pp.index_offset    = a.index_offset;
  pp.tile            = (uint32_t)pl.tile;
  pp.tiles_per_row   = (uint32_t)pl.tiles_per_row;
  pp.tiles_per_chunk = (uint32_t)pl.tiles_per_chunk;
  pp.chunks_per_row  = (uint32_t)pl.chunks_per_row;
  pp.chunks_per_slab = (uint32_t)pl.chunks_per_slab;
  pp.slabs_per_row   = (uint32_t)pl.slabs_per_row;
  pp.xform           = pl.dt.xform;
  pp.rank_by_add     = rank_by_add_on_current_device();
  pp.done_flag       = run.done_flag;
  pp.go_flag         = run.go_flag;
  pp.digit_base      = run.digit_base;
  pp.n_rows          = (uint32_t)pl.rows;
  pp.key_buf[0]      = S + pl.off_keys[0];
  pp.key_buf[1]      = S + pl.off_keys[1];
  pp.pay_buf[0]      = PAY != PAY_NONE ? S + pl.off_pay[0] : nullptr;
  pp.pay_buf[1]      = PAY != PAY_NONE ? S + pl.off_pay[1] : nullptr;

  // where the pass that writes the result puts it
  void* final_keys = nullptr;
  void* final_pay  = nullptr;
  if (pl.gather_values)
    final_keys = nullptr;
  else if (alias_keys)
    final_keys = S + pl.off_keys[0];
  else
    final_keys = write_keys_last ? vout : run.keys_for_fixup;
  if (PAY != PAY_NONE) {
    if (pl.gather_values)
      final_pay = S + pl.off_gather_idx;
    else if (alias_pay)
      final_pay = S + pl.off_pay[0];
    else
      final_pay = iout;
  }

  const void* cur_keys = vin;
  const void* cur_pay  = iin;
  for (int pass = 0; pass < pl.n_passes; ++pass) {
    const bool first = pass == 0, last = pass == pl.n_passes - 1;
    void* dst_keys;
    void* dst_pay = nullptr;
    if (last) {
      dst_keys = final_keys;
      dst_pay  = final_pay;
    } else {
      dst_keys = S + pl.off_keys[pass & 1];
      if (PAY != PAY_NONE) dst_pay = S + pl.off_pay[pass & 1];
    }

    pp.keys_in  = cur_keys;
    pp.keys_out = dst_keys;
    pp.pay_in   = cur_pay;
    pp.pay_out  = dst_pay;
    pp.shift    = (pass + run.digit_base) * RADIX_BITS;
    {
      uint8_t* side = (pl.side_band || pl.side_adaptive) ? reinterpret_cast<uint8_t*>(S + pl.off_digits) : nullptr;
      pp.digits_in  = first ? nullptr : side;  // written by the pass before
      pp.digits_out = last ? nullptr : side;   // read by the next upsweep, which runs after this scatter
      pp.side_flags = pl.side_adaptive ? reinterpret_cast<uint32_t*>(S + pl.off_side_flag) : nullptr;
    }
    pp.pass     = pass;
    pp.n_passes = pl.n_passes;
    {
      unsigned long long* bits = reinterpret_cast<unsigned long long*>(S + pl.off_key_bits);
      pp.key_bits_out = (pl.skip_dead_passes && first) ? bits : nullptr;
      pp.key_bits     = pl.skip_dead_passes ? bits : nullptr;  // complete once the first upsweep has run
      pp.early_last   = pl.early_last;
    }
    pp.slab_tot = reinterpret_cast<unsigned long long*>(S + pl.off_slab_tot + (pass & 1) * pl.slab_tot_bytes);
    pp.slab_tot_next =
      last ? nullptr
           : reinterpret_cast<unsigned long long*>(S + pl.off_slab_tot + ((pass + 1) & 1) * pl.slab_tot_bytes);
    launch_pass<KeyT, PAY>(L, pl, first, last, pp);
    if (pass >= 1 && pass <= pl.early_last && !last) {
      // If no key varies in any digit after this one, this pass writes the result: the same
      // scatter in its last-pass form, which returns at once otherwise (as the form above
      // does in that case).
      PassParams pe    = pp;
      pe.keys_out      = final_keys;
      pe.pay_out       = final_pay;
      pe.digits_out    = nullptr;
      pe.slab_tot_next = nullptr;
      launch_downsweep<KeyT, PAY>(L, pl, K_DOWN_LAST, false, true, pe);
    }

    if constexpr (is_float_width<KeyT>() && PAY == PAY_NONE) {
      if (pl.specials && first) {
        // per-row totals and exclusive offsets of the zero / NaN counts of the upsweep
        L.run(K_SPECIAL_SCAN, [&] {
          hipLaunchKernelGGL(special_scan_kernel, dim3((unsigned)pl.rows), dim3(256), 0, L.stream,
                             special_blk, special_row,
                             (uint32_t)(pl.chunks_per_row * (kUpsweepThreads / 64)));
        });
      }
      if (pl.specials && !specials_late && pass == pl.n_passes - 2) {
        // The buffer the last pass will not read is free now, and the input is still intact
        // (only the last pass writes values_out, which may alias values_in): collect the
        // original zeros / NaNs there, in input order.
        KeyT* side = reinterpret_cast<KeyT*>(S + pl.off_keys[(pl.n_passes - 1) & 1]);
        L.run(K_SPECIAL_COLLECT, [&] {
          hipLaunchKernelGGL((special_collect_kernel<KeyT, kUpsweepThreads>),
                             dim3((unsigned)pl.n_chunks), dim3(kUpsweepThreads), 0, L.stream,
                             reinterpret_cast<const KeyT*>(vin), side, special_blk, special_row,
                             (uint64_t)pl.row_len, (uint32_t)pl.chunks_per_row,
                             (uint64_t)pl.tiles_per_chunk * pl.tile, false);
        });
      }
    }
    cur_keys = dst_keys;
    cur_pay  = dst_pay;
  }

  if (alias_keys) launch_copy(L, K_COPY, vout, S + pl.off_keys[0], pl.volume * eb);
  if (alias_pay) launch_copy(L, K_COPY, iout, S + pl.off_pay[0], pl.volume * pay_bytes);

  if constexpr (sizeof(KeyT) == 8) {
    if (run.upper_first) {
      // the result is in order of the upper digits: runs of equal upper digits by the whole key
      UpperFirstParams up{};
      up.volume  = pl.volume;
      up.row_len = pl.row_len;
      up.xform    = pl.dt.xform;
      up.low_bits = RADIX_BITS * run.digit_base;
      up.flags    = reinterpret_cast<uint32_t*>(S + pl.off_uf_flags);
      up.elems   = final_keys;
      up.pos     = PAY != PAY_NONE ? reinterpret_cast<int64_t*>(final_pay) : nullptr;
      const size_t per = (size_t)UF_FIX_NT * UF_FIX_IPT;
      const size_t cpr = (pl.row_len + per - 1) / per;
      L.run(K_UF_FIXUP, [&] {
        if (PAY != PAY_NONE)
          hipLaunchKernelGGL((upper_first_fixup_kernel<KeyT, true>), dim3((unsigned)(pl.rows * cpr)), dim3(UF_FIX_NT), 0,
                             L.stream, up, (uint32_t)cpr);
        else
          hipLaunchKernelGGL((upper_first_fixup_kernel<KeyT, false>), dim3((unsigned)(pl.rows * cpr)), dim3(UF_FIX_NT),
                             0, L.stream, up, (uint32_t)cpr);
      });
    }
  }

  if constexpr (is_float_width<KeyT>() && PAY == PAY_NONE) {
    if (specials_late) {
      L.run(K_SPECIAL_COLLECT, [&] {
        hipLaunchKernelGGL((special_collect_kernel<KeyT, kUpsweepThreads>), dim3((unsigned)pl.n_chunks),
                           dim3(kUpsweepThreads), 0, L.stream, reinterpret_cast<const KeyT*>(vin),
                           reinterpret_cast<KeyT*>(vout), special_blk, special_row, (uint64_t)pl.row_len,
                           (uint32_t)pl.chunks_per_row, (uint64_t)pl.tiles_per_chunk * pl.tile, true);
      });
    } else if (pl.specials) {
      const KeyT* side = reinterpret_cast<const KeyT*>(S + pl.off_keys[(pl.n_passes - 1) & 1]);
      size_t bpr       = (pl.row_len + 16383) / 16384;
      if (bpr > 1024) bpr = 1024;
      L.run(K_SPECIAL_PATCH, [&] {
        hipLaunchKernelGGL((special_patch_kernel<KeyT>), dim3((unsigned)(pl.rows * bpr)), dim3(256),
                           0, L.stream, side, reinterpret_cast<KeyT*>(vout), special_row,
                           (uint64_t)pl.row_len, (uint32_t)bpr);
      });
    }
  }
}

template <typename KeyT>
static void radix_sort_dispatch_pay(Launcher& L, const Plan& pl, const SortArgs& a)
{
  switch (pl.pay) {
    case PAY_NONE: radix_sort_rows<KeyT, PAY_NONE>(L, pl, a); break;
    case PAY_IDX32: radix_sort_rows<KeyT, PAY_IDX32>(L, pl, a); break;
    default: radix_sort_rows<KeyT, PAY_I64>(L, pl, a); break;
  }
}

static void radix_sort_dispatch(Launcher& L, const Plan& pl, const SortArgs& a)
{
  switch (pl.dt.bytes) {
    case 1: radix_sort_dispatch_pay<uint8_t>(L, pl, a); break;
    case 2: radix_sort_dispatch_pay<uint16_t>(L, pl, a); break;
    case 4: radix_sort_dispatch_pay<uint32_t>(L, pl, a); break;
    case 8: radix_sort_dispatch_pay<uint64_t>(L, pl, a); break;
    default: radix_sort_dispatch_pay<u128>(L, pl, a); break;
  }
}

// ---------------------------------------------------------------------------------------
// one row through sample -> count -> scatter -> sort the bins (bucket.hpp)
// ---------------------------------------------------------------------------------------
template <typename KeyT, int PAY>
static void bucket_sort_row(Launcher& L, const Plan& pl, const SortArgs& a, int attempt)
{
  char* S = a.scratch;
  BucketParams p{};
  p.attempt         = attempt;
  p.flags           = attempt ? reinterpret_cast<uint32_t*>(S + pl.off_bk_flags) : nullptr;
  p.keys_in         = a.values_in;
  p.pay_in          = a.indices_in;
  p.keys_out        = a.values_out;
  p.pay_out         = a.indices_out;
  p.buf_keys[0]     = S + pl.off_keys[0];
  p.buf_keys[1]     = S + pl.off_keys[1];
  p.buf_pay[0]      = PAY != PAY_NONE ? S + pl.off_pay[0] : nullptr;
  p.buf_pay[1]      = PAY != PAY_NONE ? S + pl.off_pay[1] : nullptr;
  p.splitters       = S + pl.off_bk_splitters;
  p.slab_tot        = reinterpret_cast<uint32_t*>(S + pl.off_bk_slab_tot);
  p.chunk_hist      = reinterpret_cast<uint32_t*>(S + pl.off_bk_chunk_hist);
  p.bin_start       = reinterpret_cast<uint32_t*>(S + pl.off_bk_bin_start);
  p.chunk_range     = reinterpret_cast<unsigned long long*>(S + pl.off_bk_chunk_range);
  p.key_range       = reinterpret_cast<unsigned long long*>(S + pl.off_bk_key_range);
  p.n               = (uint32_t)pl.row_len;
  p.n_split         = pl.bk_split;
  p.oversample      = pl.bk_oversample;
  p.tile            = pl.bk_tile;
  p.tiles_per_chunk = pl.bk_tiles_per_chunk;
  p.n_chunks        = pl.bk_chunks;
  p.chunks_per_slab = (uint32_t)kChunksPerSlab;
  p.n_slabs         = pl.bk_slabs;
  p.cap             = pl.bk_cap;
  p.index_offset    = a.index_offset;
  p.xform           = pl.dt.xform;
  p.keys_travel     = pl.dt.xform == XF_COMPLEX ? 1 : 0;
  p.rank_by_add     = rank_by_add_on_current_device();
  p.direct_equal    = (a.values_out == nullptr || a.values_out != a.values_in) &&
                      (a.indices_out == nullptr || a.indices_out != a.indices_in);
  constexpr int IPT = bucket_sort_ipt(sizeof(KeyT), PAY);
  const unsigned rows = (unsigned)pl.rows;
  L.run(K_BUCKET_PLAN, [&] {
    if ((pl.bk_split + 1) * pl.bk_oversample <= (uint32_t)BK_PLAN_NT * BK_PLAN_IPT)
      hipLaunchKernelGGL((bucket_plan_kernel<KeyT, BK_PLAN_IPT>), dim3(rows), dim3(BK_PLAN_NT), 0, L.stream, p);
    else
      hipLaunchKernelGGL((bucket_plan_kernel<KeyT, 2 * BK_PLAN_IPT>), dim3(rows), dim3(BK_PLAN_NT), 0, L.stream, p);
  });
  L.run(K_BUCKET_COUNT, [&] {
    if (attempt)
      hipLaunchKernelGGL((bucket_count_kernel<KeyT, false>), dim3(pl.bk_chunks, rows), dim3(BK_COUNT_NT), 0, L.stream, p);
    else
      hipLaunchKernelGGL((bucket_count_kernel<KeyT, true>), dim3(pl.bk_chunks, rows), dim3(BK_COUNT_NT), 0, L.stream, p);
  });
  L.run(K_BUCKET_SCATTER, [&] {
    constexpr int LARGE = bucket_scatter_ipt_large(sizeof(KeyT), PAY);
    if (pl.bk_tile == (uint32_t)BK_NT * kBucketScatterIptSmall)
      hipLaunchKernelGGL((bucket_scatter_kernel<KeyT, PAY, kBucketScatterIptSmall>), dim3(pl.bk_chunks, rows),
                         dim3(BK_NT), 0, L.stream, p);
    else
      hipLaunchKernelGGL((bucket_scatter_kernel<KeyT, PAY, LARGE>), dim3(pl.bk_chunks, rows), dim3(BK_NT), 0,
                         L.stream, p);
  });
  L.run(K_BUCKET_SORT, [&] {
    const dim3 grid(attempt ? BK_SLOTS : pl.bk_split + 1, rows);
    hipLaunchKernelGGL((bucket_sort_kernel<KeyT, PAY, IPT>), grid, dim3(BK_NT), 0, L.stream, p);
  });
}

template <typename KeyT>
static void bucket_sort_dispatch_pay(Launcher& L, const Plan& pl, const SortArgs& a)
{
  switch (pl.pay) {
    case PAY_NONE: bucket_sort_row<KeyT, PAY_NONE>(L, pl, a); break;
    case PAY_IDX32: bucket_sort_row<KeyT, PAY_IDX32>(L, pl, a); break;
    default: bucket_sort_row<KeyT, PAY_I64>(L, pl, a); break;
  }
}

static void bucket_sort_dispatch(Launcher& L, const Plan& pl, const SortArgs& a)
{
  switch (pl.dt.bytes) {
    case 1: bucket_sort_dispatch_pay<uint8_t>(L, pl, a); break;
    case 2: bucket_sort_dispatch_pay<uint16_t>(L, pl, a); break;
    case 4: bucket_sort_dispatch_pay<uint32_t>(L, pl, a); break;
    default: bucket_sort_dispatch_pay<uint64_t>(L, pl, a); break;
  }
}

// ---------------------------------------------------------------------------------------
// counting sort of one long row of 2-byte elements (values only)
// ---------------------------------------------------------------------------------------
static void count16_sort(Launcher& L, const Plan& pl, const SortArgs& a)
{
  char* S             = a.scratch;
  const uint16_t* vin = reinterpret_cast<const uint16_t*>(a.values_in);
  uint16_t* vout      = reinterpret_cast<uint16_t*>(a.values_out);
  auto* special_row   = reinterpret_cast<unsigned long long*>(S + pl.off_special_ctr);
  auto* special_blk   = reinterpret_cast<unsigned long long*>(S + pl.off_special_blk);
  auto* ghist         = reinterpret_cast<unsigned long long*>(S + pl.off_c16_hist);
  auto* prefix        = reinterpret_cast<unsigned long long*>(S + pl.off_c16_prefix);
  uint16_t* side      = reinterpret_cast<uint16_t*>(S + pl.off_keys[0]);
  const uint64_t n    = pl.row_len;

  // special counters and key counters are adjacent in the scratch layout
  launch_zero(L, S + pl.off_special_ctr,
              pl.off_c16_hist - pl.off_special_ctr + (size_t)C16_BINS * sizeof(unsigned long long));
  const dim3 hgrid((unsigned)(pl.c16_chunks * C16_SLICES));
  L.run(K_COUNT16_HIST, [&] {
    if (pl.specials)
      hipLaunchKernelGGL((count16_hist_kernel<true>), hgrid, dim3(C16_HIST_NT), 0, L.stream, vin, n,
                         (uint64_t)pl.c16_chunk_len, ghist, special_blk);
    else
      hipLaunchKernelGGL((count16_hist_kernel<false>), hgrid, dim3(C16_HIST_NT), 0, L.stream, vin, n,
                         (uint64_t)pl.c16_chunk_len, ghist, special_blk);
  });
  L.run(K_COUNT16_SCAN, [&] {
    hipLaunchKernelGGL(count16_scan_kernel, dim3(1), dim3(1024), 0, L.stream, ghist, prefix,
                       (unsigned long long)n, pl.dt.xform, pl.specials ? special_row : nullptr);
  });
  if (pl.specials) {
    // the input is still intact here (values_out may alias it): collect the original zeros
    // and NaNs in input order before anything is written
    L.run(K_SPECIAL_SCAN, [&] {
      hipLaunchKernelGGL(special_scan_kernel, dim3(1), dim3(256), 0, L.stream, special_blk,
                         special_row, (uint32_t)(pl.c16_chunks * (C16_HIST_NT / 64)));
    });
    L.run(K_SPECIAL_COLLECT, [&] {
      hipLaunchKernelGGL((special_collect_kernel<uint16_t, C16_HIST_NT>), dim3((unsigned)pl.c16_chunks),
                         dim3(C16_HIST_NT), 0, L.stream, vin, side, special_blk, special_row, n,
                         (uint32_t)pl.c16_chunks, (uint64_t)pl.c16_chunk_len, false);
    });
  }
  constexpr uint64_t span = (uint64_t)C16_FILL_NT * C16_FILL_VEC * 8;
  L.run(K_COUNT16_FILL, [&] {
    hipLaunchKernelGGL(count16_fill_kernel, dim3((unsigned)((n + span - 1) / span)), dim3(C16_FILL_NT),
                       0, L.stream, vout, n, prefix, pl.dt.xform);
  });
  if (pl.specials) {
    size_t bpr = (pl.row_len + 16383) / 16384;
    if (bpr > 1024) bpr = 1024;
    L.run(K_SPECIAL_PATCH, [&] {
      hipLaunchKernelGGL((special_patch_kernel<uint16_t>), dim3((unsigned)bpr), dim3(256), 0, L.stream,
                         side, vout, special_row, n, (uint32_t)bpr);
    });
  }
}

// counting sort of one long row of 1-byte elements (values only)
static void count8_sort(Launcher& L, const Plan& pl, const SortArgs& a)
{
  auto* ghist      = reinterpret_cast<unsigned long long*>(a.scratch + pl.off_c16_hist);
  const uint64_t n = pl.row_len;
  launch_zero(L, ghist, 256 * sizeof(unsigned long long));
  uint64_t hb = (n / 16 + C8_NT - 1) / C8_NT;  // one 16-byte load per thread and round
  if (hb > 2048) hb = 2048;
  if (hb < 1) hb = 1;
  L.run(K_COUNT8_HIST, [&] {
    hipLaunchKernelGGL(count8_hist_kernel, dim3((unsigned)hb), dim3(C8_NT), 0, L.stream,
                       reinterpret_cast<const uint8_t*>(a.values_in), n, ghist);
  });
  uint64_t fb = (n + (uint64_t)C8_NT * 64 - 1) / ((uint64_t)C8_NT * 64);  // spans of the fill
  if (fb > 4096) fb = 4096;
  L.run(K_COUNT8_FILL, [&] {
    hipLaunchKernelGGL(count8_fill_kernel, dim3((unsigned)fb), dim3(C8_NT), 0, L.stream,
                       reinterpret_cast<uint8_t*>(a.values_out), n, ghist, pl.dt.xform);
  });
}

// ---------------------------------------------------------------------------------------
// partition / argpartition by selection: pivot by radix select, then one three-way split
// ---------------------------------------------------------------------------------------
struct PartLayout {
  Plan pl;              // geometry of the split pass (and the plan of the fallback sort)
  bool select = false;  // false: the ordinary sort is used (it is a valid partition)
  size_t off_pivot = 0, off_kleft = 0, off_ghist = 0, off_stage = 0;
  // radix select: per-row state and candidate counts, the candidate keys of every row with
  // the chunks they came from, what every chunk counted in every pass
  size_t off_sel_state = 0, off_cand_from = 0, off_cand_n = 0, off_cand = 0, off_cand_chunk = 0, cand_cap = 0;
  size_t off_cand_less_eq = 0, off_pass_hist = 0, zeroed_end = 0;
  size_t off_n_equal = 0, off_above_max = 0, off_chunk_cls = 0, off_chunk_off = 0;
  size_t total = 0;
};

// select_only: the layout of misort_select, which finds the key and does not move the row
static int partition_layout(int dtype, size_t volume, size_t sort_dim_size, bool want_indices,
                            long long kth, PartLayout& u, bool select_only = false)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return fail(MISORT_ERR_DTYPE, "unknown dtype code");
  // (the selection walks the chunks of the radix plan)
  PlanOptions radix_only;
  radix_only.bucket_path     = 0;
  radix_only.low_cardinality = 0;
  radix_only.upper_first     = 0;
  int rc = make_plan(dtype, volume, sort_dim_size, want_indices, false, u.pl, radix_only);
  if (rc != MISORT_OK) return rc;
  // 1- and 2-byte values are counted, which beats selecting; their positions are selected
  u.select = u.pl.strategy == S_RADIX && u.pl.pay != PAY_I64 && kth >= 0 &&
             (unsigned long long)kth < u.pl.row_len && (want_indices || dt.bytes > 2);
  if (!u.select) {
    // plan of the sort that is actually run
    Plan sp;
    rc = make_plan(dtype, volume, sort_dim_size, want_indices, false, sp);
    if (rc != MISORT_OK) return rc;
    u.pl    = sp;
    u.total = sp.total;
    return MISORT_OK;
  }
  size_t off = 0;
  auto take  = [&](size_t bytes) {
    const size_t o = off;
    off += align_up(bytes, 256);
    return o;
  };
  Plan& pl          = u.pl;
  u.off_pivot       = take(pl.rows * 16);
  u.off_kleft       = take(pl.rows * sizeof(unsigned long long));
  u.off_ghist       = take(pl.rows * RADIX * sizeof(unsigned long long));
  u.off_cand_less_eq = take(pl.n_chunks * 2 * sizeof(uint32_t));  // cleared together with the counters before it
  u.zeroed_end      = off;
  u.off_chunk_cls   = take(pl.n_chunks * 4 * sizeof(uint32_t));
  u.off_chunk_off   = take(pl.n_chunks * 4 * sizeof(unsigned long long));
  u.off_pass_hist   = take((size_t)dt.bytes * pl.n_chunks * RADIX * sizeof(uint32_t));
  u.off_sel_state   = take(pl.rows * sizeof(uint32_t));
  u.off_n_equal     = take(pl.rows * sizeof(unsigned long long));
  u.off_above_max   = take(pl.rows * 3 * sizeof(unsigned long long));
  u.off_cand_from   = take(pl.rows * sizeof(uint32_t));
  u.off_cand_n      = take(pl.rows * sizeof(unsigned long long));
  u.cand_cap        = pl.row_len / 8 + 1;  // keys that still match, once they are this few
  u.off_cand        = take(pl.rows * u.cand_cap * pl.dt.bytes);
  u.off_cand_chunk  = take(pl.rows * u.cand_cap * sizeof(uint32_t));
  if (!select_only && !want_indices) u.off_stage = take(pl.volume * pl.dt.bytes);  // values when in == out
  u.total = off;
  return MISORT_OK;
}

// The selection proper: after it sp.prefix holds the kth key of every row.  neighbours: the
// rows' above_max words are wanted (select_init_kernel sets them up).
template <typename KeyT>
static SelectParams<KeyT> run_selection(Launcher& L, const PartLayout& u, const void* vin, long long kth,
                                        char* S, bool neighbours)
{
  const Plan& pl = u.pl;
  SelectParams<KeyT> sp{};
  sp.in              = reinterpret_cast<const KeyT*>(vin);
  sp.row_len         = pl.row_len;
  sp.chunk_len       = (uint64_t)pl.tiles_per_chunk * pl.tile;
  sp.chunks_per_row  = (uint32_t)pl.chunks_per_row;
  sp.n_chunks        = (uint32_t)pl.n_chunks;
  sp.n_passes        = (uint32_t)sizeof(KeyT);
  sp.xform           = pl.dt.xform;
  sp.prefix          = reinterpret_cast<KeyT*>(S + u.off_pivot);
  sp.kleft           = reinterpret_cast<unsigned long long*>(S + u.off_kleft);
  sp.ghist           = reinterpret_cast<unsigned long long*>(S + u.off_ghist);
  sp.pass_hist       = reinterpret_cast<uint32_t*>(S + u.off_pass_hist);
  sp.state           = reinterpret_cast<uint32_t*>(S + u.off_sel_state);
  sp.cand_from       = reinterpret_cast<uint32_t*>(S + u.off_cand_from);
  sp.cand            = reinterpret_cast<KeyT*>(S + u.off_cand);
  sp.cand_chunk      = reinterpret_cast<uint32_t*>(S + u.off_cand_chunk);
  sp.cand_n          = reinterpret_cast<unsigned long long*>(S + u.off_cand_n);
  sp.cand_cap        = u.cand_cap;
  sp.n_equal         = reinterpret_cast<unsigned long long*>(S + u.off_n_equal);
  sp.above_max       = neighbours ? reinterpret_cast<unsigned long long*>(S + u.off_above_max) : nullptr;
  sp.cand_less_eq    = reinterpret_cast<uint32_t*>(S + u.off_cand_less_eq);
  sp.chunk_cls       = reinterpret_cast<uint32_t*>(S + u.off_chunk_cls);
  sp.chunk_off       = reinterpret_cast<unsigned long long*>(S + u.off_chunk_off);
  const dim3 grid((unsigned)pl.n_chunks);
  const dim3 rgrid((unsigned)pl.rows);

  launch_zero(L, sp.ghist, u.zeroed_end - u.off_ghist);
  L.run(K_SELECT_INIT, [&] {
    hipLaunchKernelGGL((select_init_kernel<KeyT>), dim3((unsigned)((pl.rows + 255) / 256)), dim3(256), 0,
                       L.stream, sp, (uint32_t)pl.rows, (unsigned long long)kth);
  });
  int pass = 0;
  for (int shift = (int)sizeof(KeyT) * 8 - 8; shift >= 0; shift -= 8, ++pass) {
    L.run(K_SELECT_HIST, [&] {
      hipLaunchKernelGGL((select_hist_kernel<KeyT>), grid, dim3(SEL_NT), 0, L.stream, sp, pass, shift);
    });
    L.run(K_SELECT_PICK, [&] {
      hipLaunchKernelGGL((select_pick_kernel<KeyT>), rgrid, dim3(RADIX), 0, L.stream, sp, pass, shift);
    });
  }
  return sp;
}

// partition / argpartition: the selection, then the split around the key it found.  Give
// values_out (which receives the values as they came in) or pos_out.
template <typename KeyT>
static void partition_select_rows(Launcher& L, const PartLayout& u, const void* vin, void* values_out,
                                  int64_t* pos_out, long long kth, int64_t index_offset, char* S)
{
  const Plan& pl              = u.pl;
  const SelectParams<KeyT> sp = run_selection<KeyT>(L, u, vin, kth, S, false);
  const dim3 grid((unsigned)pl.n_chunks);
  // where the split puts the keys of every chunk, from what the passes above counted per chunk
  L.run(K_SELECT_COUNTS, [&] {
    hipLaunchKernelGGL((select_cand_counts_kernel<KeyT>), grid, dim3(SEL_NT), 0, L.stream, sp);
    hipLaunchKernelGGL((select_chunk_counts_kernel<KeyT>), grid, dim3(RADIX), 0, L.stream, sp);
    hipLaunchKernelGGL((select_chunk_offsets_kernel<KeyT>), dim3((unsigned)pl.rows), dim3(256), 0, L.stream, sp);
  });
  constexpr int NT = 1024, IPT = sizeof(KeyT) >= 16 ? 4 : 8;
  L.run(K_SPLIT, [&] {
    if (pos_out) {
      hipLaunchKernelGGL((select_split_kernel<KeyT, true, NT, IPT>), grid, dim3(NT), 0, L.stream, sp, nullptr,
                         pos_out, index_offset);
    } else {
      if constexpr (sizeof(KeyT) > 2)  // (values of 1 and 2 bytes are counted, not selected)
        hipLaunchKernelGGL((select_split_kernel<KeyT, false, NT, IPT>), grid, dim3(NT), 0, L.stream, sp,
                           reinterpret_cast<KeyT*>(values_out), nullptr, index_offset);
    }
  });
}

// misort_select: the selection, one more read of the row for the neighbours of the kth key,
// and the values written out
template <typename KeyT>
static void select_rows(Launcher& L, const PartLayout& u, const void* vin, long long kth, void* kth_out,
                        void* next_out, void* max_out, char* S)
{
  const Plan& pl              = u.pl;
  const SelectParams<KeyT> sp = run_selection<KeyT>(L, u, vin, kth, S, true);
  if (next_out)
    L.run(K_SELECT_NEIGHBOURS, [&] {
      hipLaunchKernelGGL((select_above_kernel<KeyT, true>), dim3((unsigned)pl.n_chunks), dim3(SEL_NT), 0,
                         L.stream, sp);
      hipLaunchKernelGGL((select_above_kernel<KeyT, false>), dim3((unsigned)pl.n_chunks), dim3(SEL_NT), 0,
                         L.stream, sp);
    });
  L.run(K_SELECT_EMIT, [&] {
    hipLaunchKernelGGL((select_emit_kernel<KeyT>), dim3((unsigned)((pl.rows + 255) / 256)), dim3(256), 0,
                       L.stream, sp, (uint32_t)pl.rows, reinterpret_cast<KeyT*>(kth_out),
                       reinterpret_cast<KeyT*>(next_out), reinterpret_cast<KeyT*>(max_out));
  });
}

// ---------------------------------------------------------------------------------------
// top level
// ---------------------------------------------------------------------------------------
static int run_sort(Launcher& L, int dtype, const void* values_in, void* values_out,
                    const int64_t* indices_in, int64_t* indices_out, size_t volume,
                    size_t sort_dim_size, int64_t index_offset, void* scratch, size_t scratch_bytes,
                    const PlanOptions& opt = PlanOptions{}, bool canonical_values = false)
{
  Plan pl;
  const bool argsort = indices_out != nullptr;
  int rc = make_plan(dtype, volume, sort_dim_size, argsort, indices_in != nullptr, pl, opt);
  if (rc != MISORT_OK) return rc;
  if (pl.strategy == S_EMPTY) return MISORT_OK;

  if (!values_in) return fail(MISORT_ERR_NULL, "values_in is NULL");
  if (!argsort && !values_out) return fail(MISORT_ERR_NULL, "values_out is NULL for a keys-only sort");
  if (!argsort && indices_in) return fail(MISORT_ERR_NULL, "indices_in given without indices_out");
  if (!scratch) return fail(MISORT_ERR_NULL, "scratch is NULL");
  if (scratch_bytes < pl.total) {
    char msg[128];
    snprintf(msg, sizeof msg, "scratch too small: %zu bytes given, %zu needed", scratch_bytes,
             pl.total);
    return fail(MISORT_ERR_SCRATCH, msg);
  }
  const size_t eb = pl.dt.bytes;
  auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (misaligned(values_in, eb) || (values_out && misaligned(values_out, eb)))
    return fail(MISORT_ERR_ALIGN, "values pointer not aligned to the element size");
  if ((indices_in && misaligned(indices_in, 8)) || (indices_out && misaligned(indices_out, 8)))
    return fail(MISORT_ERR_ALIGN, "indices pointer not aligned to 8 bytes");
  if (misaligned(scratch, 256)) return fail(MISORT_ERR_ALIGN, "scratch not aligned to 256 bytes");
  if (argsort && values_out && values_out == values_in)
    return fail(MISORT_ERR_ALIAS,
                "argsort: values_out must be NULL or a buffer distinct from values_in");
  auto overlaps = [&](const void* p, size_t bytes) {
    if (!p) return false;
    const char* b = reinterpret_cast<const char*>(p);
    const char* s = reinterpret_cast<const char*>(scratch);
    return b < s + pl.total && s < b + bytes;
  };
  if (overlaps(values_in, volume * eb) || overlaps(values_out, volume * eb) ||
      overlaps(indices_in, volume * 8) || overlaps(indices_out, volume * 8))
    return fail(MISORT_ERR_ALIAS, "scratch overlaps an input or output buffer");

  SortArgs a{values_in, values_out, indices_in, indices_out, index_offset,
             reinterpret_cast<char*>(scratch)};

  // argsort with values_out: the index sort runs with values_out = NULL, then the sorted
  // elements are gathered, which keeps the original bit patterns of zeros and NaNs.
  // (With a caller-filled payload there are no positions to gather by: the last pass
  // writes the keys back through the inverse transform instead.)
  SortArgs core = a;
  // (canonical_values: the caller only compares the sorted values through their keys, so the
  // last pass may write them through the inverse key transform, which maps -0 to +0 and
  // every NaN to one NaN; not for complex elements, whose NaN tiers have no inverse)
  if (pl.values_as_payload) {  // the elements are the payload of their own keys
    core.indices_in  = reinterpret_cast<const int64_t*>(values_in);
    core.indices_out = reinterpret_cast<int64_t*>(values_out);
    core.values_out  = nullptr;
  }
  const bool gather_sorted =
    argsort && values_out && !indices_in && !(canonical_values && pl.dt.xform != XF_COMPLEX);
  if (gather_sorted) core.values_out = nullptr;
  if (argsort && values_out && indices_in && pl.dt.xform == XF_COMPLEX)
    return fail(MISORT_ERR_UNSUPPORTED,
                "complex argsort with both a caller payload and values_out is not supported");

  switch (pl.strategy) {
    case S_ROW_WAVE:
    case S_ROW_BLOCK:
      launch_rowsort(L, pl.strategy == S_ROW_WAVE ? K_ROWSORT_WAVE : K_ROWSORT_BLOCK,
                     pl.strategy == S_ROW_WAVE, pl.dt.bytes, pl.dt.xform, pl.pay, core.values_in,
                     core.values_out, core.indices_in, core.indices_out, pl.rows, pl.row_len,
                     index_offset);
      break;
    case S_COUNT16: count16_sort(L, pl, core); break;
    case S_COUNT8: count8_sort(L, pl, core); break;
    case S_BUCKET: bucket_sort_dispatch(L, pl, core); break;
    case S_RADIX:
      radix_sort_dispatch(L, pl, core);
      if (pl.gather_values) {
        // complex keys-only: elements gathered by sorted position
        const void* src = values_in;
        if (values_in == values_out) {
          launch_copy(L, K_COPY, a.scratch + pl.off_gather_src, values_in, volume * eb);
          src = a.scratch + pl.off_gather_src;
        }
        launch_gather(L, K_GATHER, eb, src, values_out,
                      reinterpret_cast<const int64_t*>(a.scratch + pl.off_gather_idx), pl.rows,
                      pl.row_len, index_offset);
      }
      break;
    default: break;
  }
  if (gather_sorted)
    launch_gather(L, K_GATHER, eb, values_in, values_out, indices_out, pl.rows, pl.row_len,
                  index_offset);
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

}  // namespace misort

// ---------------------------------------------------------------------------------------
// scratch that belongs to the library: misort_local_static sorts without any buffer from
// the caller beyond the inputs and outputs, and without allocating.  One copy of the array
// exists per GPU; in host code its name is only a handle for hipGetSymbolAddress.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char misort_static_scratch[MISORT_STATIC_SCRATCH_BYTES];

namespace misort {

static std::atomic<void*> g_static_scratch_ptr[kMaxDevices];

// Device address of misort_static_scratch on the current GPU, looked up once per GPU.  A
// stream that belongs to another GPU than the current one is refused: its kernels would be
// handed the current GPU's copy of the buffer.
static int static_scratch_address(void** out, hipStream_t stream = nullptr)
{
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("hipGetDevice: ") + hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MISORT_ERR_UNSUPPORTED, "device ordinal above 63");
  if (stream) {
    hipDevice_t sdev = -1;
    if (hipStreamGetDevice(stream, &sdev) == hipSuccess && (int)sdev != dev)
      return fail(MISORT_ERR_UNSUPPORTED, "misort_local_static: the stream belongs to another GPU than the current one");
    (void)hipGetLastError();
  }
  void* p = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(misort_static_scratch));
    if (e != hipSuccess || !p)
      return fail(MISORT_ERR_RUNTIME, std::string("hipGetSymbolAddress: ") + hipGetErrorString(e));
    g_static_scratch_ptr[dev].store(p, std::memory_order_release);  // same value from any thread
  }
  *out = p;
  return MISORT_OK;
}

}  // namespace misort

using namespace misort;

extern "C" {

int misort_version(void) { return 100; }

size_t misort_dtype_size(int dtype)
{
  DtypeInfo d;
  return dtype_info(dtype, d) ? (size_t)d.bytes : 0;
}

const char* misort_last_error(void) { return g_last_error.c_str(); }

size_t misort_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                            int has_indices_in)
{
  Plan pl;
  if (make_plan(dtype, volume, sort_dim_size, argsort != 0, has_indices_in != 0, pl) != MISORT_OK)
    return 0;
  return pl.total;
}

int misort_local(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                 int64_t* indices_out, size_t volume, size_t sort_dim_size, int /*stable*/,
                 int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream)
{
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  return run_sort(L, dtype, values_in, values_out, indices_in, indices_out, volume, sort_dim_size,
                  index_offset, scratch, scratch_bytes);
}

int misort_local_static(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                        int64_t* indices_out, size_t volume, size_t sort_dim_size, int /*stable*/,
                        int64_t index_offset, void* stream)
{
  Plan pl;
  int rc = make_plan(dtype, volume, sort_dim_size, indices_out != nullptr, indices_in != nullptr, pl);
  if (rc != MISORT_OK) return rc;
  if (pl.total > (size_t)MISORT_STATIC_SCRATCH_BYTES) {
    char msg[160];
    snprintf(msg, sizeof msg,
             "misort_local_static: this sort needs %zu bytes of scratch, the library's own buffer "
             "holds %zu; use misort_local with a caller buffer",
             pl.total, (size_t)MISORT_STATIC_SCRATCH_BYTES);
    return fail(MISORT_ERR_SCRATCH, msg);
  }
  if (pl.strategy == S_EMPTY) return MISORT_OK;
  void* own = nullptr;
  rc        = static_scratch_address(&own, reinterpret_cast<hipStream_t>(stream));
  if (rc != MISORT_OK) return rc;
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  return run_sort(L, dtype, values_in, values_out, indices_in, indices_out, volume, sort_dim_size,
                  index_offset, own, (size_t)MISORT_STATIC_SCRATCH_BYTES);
}

size_t misort_scratch_bytes_chunked(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                                    int has_indices_in, size_t target_chunks)
{
  Plan pl;
  PlanOptions opt;
  opt.target_chunks = target_chunks;
  if (make_plan(dtype, volume, sort_dim_size, argsort != 0, has_indices_in != 0, pl, opt) != MISORT_OK)
    return 0;
  return pl.total;
}

int misort_local_chunked(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                         int64_t* indices_out, size_t volume, size_t sort_dim_size, int /*stable*/,
                         int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream,
                         size_t target_chunks)
{
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  PlanOptions opt;
  opt.target_chunks = target_chunks;
  return run_sort(L, dtype, values_in, values_out, indices_in, indices_out, volume, sort_dim_size,
                  index_offset, scratch, scratch_bytes, opt);
}

static PlanOptions plan_options(const misort_options* o)
{
  PlanOptions opt;
  if (o) {
    opt.target_chunks        = o->target_chunks;
    opt.early_last_min_bytes = o->early_last_min_bytes;
    opt.bucket_path          = o->bucket_path;
    opt.bucket_bins          = o->bucket_bins;
    opt.bucket_cap           = o->bucket_cap;
    opt.low_cardinality      = o->low_cardinality;
    opt.bucket_oversample    = o->bucket_oversample;
    opt.counting_sort        = o->counting_sort;
    opt.upper_first          = o->upper_first;
  }
  return opt;
}

size_t misort_scratch_bytes_opts(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                                 int has_indices_in, const misort_options* options)
{
  Plan pl;
  if (make_plan(dtype, volume, sort_dim_size, argsort != 0, has_indices_in != 0, pl, plan_options(options)) !=
      MISORT_OK)
    return 0;
  return pl.total;
}

int misort_local_opts(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                      int64_t* indices_out, size_t volume, size_t sort_dim_size, int /*stable*/,
                      int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream,
                      const misort_options* options)
{
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  return run_sort(L, dtype, values_in, values_out, indices_in, indices_out, volume, sort_dim_size,
                  index_offset, scratch, scratch_bytes, plan_options(options));
}

int misort_init(void)
{
  void* own = nullptr;
  const int rc = static_scratch_address(&own);
  if (rc != MISORT_OK) return rc;
  (void)rank_by_add_on_current_device();
  return MISORT_OK;
}

int misort_rank_mode(void)
{
  if (rank_ballot_env()) return 2;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  return g_rank_mode[dev].load(std::memory_order_acquire);
}

int misort_local_profiled(int dtype, const void* values_in, void* values_out,
                          const int64_t* indices_in, int64_t* indices_out, size_t volume,
                          size_t sort_dim_size, int /*stable*/, int64_t index_offset, void* scratch,
                          size_t scratch_bytes, void* stream, float* kernel_ms, int* kernel_ids,
                          int max_kernels, int* n_kernels)
{
  Launcher L;
  L.stream  = reinterpret_cast<hipStream_t>(stream);
  L.profile = true;
  const int rc = run_sort(L, dtype, values_in, values_out, indices_in, indices_out, volume,
                          sort_dim_size, index_offset, scratch, scratch_bytes);
  hipError_t e = hipStreamSynchronize(L.stream);
  const int n  = (int)L.ids.size();
  if (n_kernels) *n_kernels = n;
  for (int i = 0; i < n; ++i) {
    float ms = 0.f;
    if (e == hipSuccess) hipEventElapsedTime(&ms, L.ev[2 * i], L.ev[2 * i + 1]);
    if (i < max_kernels) {
      if (kernel_ms) kernel_ms[i] = ms;
      if (kernel_ids) kernel_ids[i] = L.ids[i];
    }
    hipEventDestroy(L.ev[2 * i]);
    hipEventDestroy(L.ev[2 * i + 1]);
  }
  if (rc == MISORT_OK && e != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(e));
  return rc;
}

const char* misort_kernel_name(int kernel_id)
{
  return (kernel_id >= 0 && kernel_id < K_NUM) ? kKernelNames[kernel_id] : "";
}

int misort_describe_plan(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                         int has_indices_in, char* buf, size_t buf_bytes)
{
  return misort_describe_plan_opts(dtype, volume, sort_dim_size, argsort, has_indices_in, nullptr, buf,
                                   buf_bytes);
}

int misort_describe_plan_opts(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                              int has_indices_in, const misort_options* options, char* buf,
                              size_t buf_bytes)
{
  Plan pl;
  const int rc =
    make_plan(dtype, volume, sort_dim_size, argsort != 0, has_indices_in != 0, pl, plan_options(options));
  if (rc != MISORT_OK) return rc;
  if (!buf || buf_bytes == 0) return fail(MISORT_ERR_NULL, "buf is NULL");
  static const char* const sname[] = {"empty", "row_wave", "row_block", "radix", "count16", "count8", "bucket"};
  static const char* const pname[] = {"none", "idx32", "i64"};
  snprintf(buf, buf_bytes,
           "strategy=%s key_bytes=%d passes=%d digit_bits=%d tile=%d rows=%zu row_len=%zu "
           "chunks_per_row=%zu tiles_per_chunk=%zu payload=%s specials=%d gather=%d side_band=%d "
           "scratch=%zu",
           sname[pl.strategy], pl.dt.bytes, pl.n_passes, RADIX_BITS, pl.tile, pl.rows, pl.row_len,
           pl.chunks_per_row, pl.tiles_per_chunk, pname[pl.pay], (int)pl.specials,
           (int)pl.gather_values, pl.side_band ? 1 : (pl.side_adaptive ? 2 : 0), pl.total);
  if (pl.strategy == S_BUCKET) {
    const size_t len = strlen(buf);
    if (len + 64 < buf_bytes)
      snprintf(buf + len, buf_bytes - len, " bins=%u bin_cap=%u chunks=%u", pl.bk_split + 1, pl.bk_cap, pl.bk_chunks);
  }
  if (pl.low_card) {
    const size_t len = strlen(buf);
    if (len + 32 < buf_bytes) snprintf(buf + len, buf_bytes - len, " low_cardinality_attempt=%d", pl.low_card);
  }
  if (pl.upper_first) {
    const size_t len = strlen(buf);
    if (len + 48 < buf_bytes)
      snprintf(buf + len, buf_bytes - len, " upper_first_attempt=%d upper_digits=%d", pl.upper_first,
               8 - upper_first_digit0(pl.dt.xform, pl.row_len));
  }
  if (pl.skip_dead_passes) {
    const size_t len = strlen(buf);
    if (len + 32 < buf_bytes)
      snprintf(buf + len, buf_bytes - len, " skip_dead_passes=1%s", pl.early_last ? " early_last=1" : "");
  }
  if (pl.strategy == S_RADIX || pl.strategy == S_BUCKET) {
    // how the scatter ranks on the current GPU (decided at the first sort there or by misort_init)
    static const char* const rname[] = {"untested", "add", "ballot"};
    const size_t len = strlen(buf);
    if (len + 16 < buf_bytes) snprintf(buf + len, buf_bytes - len, " rank=%s", rname[misort_rank_mode()]);
  }
  return MISORT_OK;
}

// searchsorted with the queries sorted first: [sorted queries | their positions | scratch of the sort]
struct SearchLayout {
  size_t off_pos = 0, off_sort = 0, sort_bytes = 0, total = 0;
};
// Sorting the queries pays when there are many of them and the array is larger than the
// caches.  Measured with float32, plain / sorted first: 2^28 elements, 2^24 queries 3.81 /
// 1.18 ms, 2^20 queries 0.34 / 0.33 ms, 2^19 queries 0.15 / 0.29 ms; 2^24 elements, 2^20
// queries 0.19 / 0.11 ms.
static bool search_sorts_queries(size_t elem_bytes, size_t n, size_t m)
{
  return m >= ((size_t)1 << 20) && n * elem_bytes >= ((size_t)64 << 20);
}
static bool search_layout(int dtype, size_t m, SearchLayout& u)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return false;
  Plan pl;
  if (make_plan(dtype, m, m, true, false, pl) != MISORT_OK) return false;
  u.off_pos    = align_up(m * dt.bytes, 256);
  u.off_sort   = u.off_pos + align_up(m * sizeof(int64_t), 256);
  u.sort_bytes = pl.total;
  u.total      = u.off_sort + align_up(pl.total, 256) + 256;
  return true;
}

size_t misort_searchsorted_scratch_bytes(int dtype, size_t n, size_t m)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt) || !search_sorts_queries(dt.bytes, n, m)) return 0;
  SearchLayout u;
  return search_layout(dtype, m, u) ? u.total : 0;
}

int misort_searchsorted_ws(int dtype, const void* sorted, size_t n, const void* values, size_t m,
                           int left, int64_t* out, void* scratch, size_t scratch_bytes, void* stream)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return fail(MISORT_ERR_DTYPE, "unknown dtype code");
  if (m == 0) return MISORT_OK;
  if (!values || !out || (n != 0 && !sorted)) return fail(MISORT_ERR_NULL, "searchsorted: NULL pointer");
  auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (misaligned(values, dt.bytes) || (n != 0 && misaligned(sorted, dt.bytes)) || misaligned(out, 8))
    return fail(MISORT_ERR_ALIGN, "searchsorted: pointer not aligned to its element size");
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  const void* queries  = values;
  const int64_t* where = nullptr;
  if (scratch && search_sorts_queries(dt.bytes, n, m)) {
    SearchLayout u;
    if (!search_layout(dtype, m, u)) return fail(MISORT_ERR_UNSUPPORTED, "searchsorted: cannot plan the sort");
    if (scratch_bytes < u.total) return fail(MISORT_ERR_SCRATCH, "searchsorted: scratch too small");
    if (misaligned(scratch, 256)) return fail(MISORT_ERR_ALIGN, "scratch not aligned to 256 bytes");
    char* S      = reinterpret_cast<char*>(scratch);
    int64_t* pos = reinterpret_cast<int64_t*>(S + u.off_pos);
    const int rc = run_sort(L, dtype, values, S, nullptr, pos, m, m, 0, S + u.off_sort,
                            u.sort_bytes > 0 ? u.sort_bytes : 256, PlanOptions{}, true);
    if (rc != MISORT_OK) return rc;
    queries = S;
    where   = pos;
  }
  if (where) {
    // consecutive sorted queries per workgroup; about 2048 workgroups
    size_t per_block = (m + 2047) / 2048;
    per_block        = (per_block + SEARCH_NT - 1) / SEARCH_NT * SEARCH_NT;
    const size_t blocks = (m + per_block - 1) / per_block;
    L.run(K_SEARCHSORTED, [&] {
#define MISORT_SEARCH_CASE(RAW)                                                                    \
  hipLaunchKernelGGL((searchsorted_sorted_kernel<RAW>), dim3((unsigned)blocks), dim3(SEARCH_NT), 0, \
                     L.stream, reinterpret_cast<const RAW*>(sorted), (uint64_t)n,                 \
                     reinterpret_cast<const RAW*>(queries), (uint64_t)m, dt.xform, left, out, where, \
                     (uint64_t)per_block)
      switch (dt.bytes) {
        case 1: MISORT_SEARCH_CASE(uint8_t); break;
        case 2: MISORT_SEARCH_CASE(uint16_t); break;
        case 4: MISORT_SEARCH_CASE(uint32_t); break;
        case 8: MISORT_SEARCH_CASE(uint64_t); break;
        default: MISORT_SEARCH_CASE(u128); break;
      }
#undef MISORT_SEARCH_CASE
    });
  } else {
    size_t blocks = (m + SEARCH_NT - 1) / SEARCH_NT;
    if (blocks > 1024) blocks = 1024;
    L.run(K_SEARCHSORTED, [&] {
#define MISORT_SEARCH_CASE(RAW)                                                                    \
  hipLaunchKernelGGL((searchsorted_kernel<RAW>), dim3((unsigned)blocks), dim3(SEARCH_NT), 0, L.stream, \
                     reinterpret_cast<const RAW*>(sorted), (uint64_t)n,                           \
                     reinterpret_cast<const RAW*>(queries), (uint64_t)m, dt.xform, left, out)
      switch (dt.bytes) {
        case 1: MISORT_SEARCH_CASE(uint8_t); break;
        case 2: MISORT_SEARCH_CASE(uint16_t); break;
        case 4: MISORT_SEARCH_CASE(uint32_t); break;
        case 8: MISORT_SEARCH_CASE(uint64_t); break;
        default: MISORT_SEARCH_CASE(u128); break;
      }
#undef MISORT_SEARCH_CASE
    });
  }
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

int misort_searchsorted(int dtype, const void* sorted, size_t n, const void* values, size_t m,
                        int left, int64_t* out, void* stream)
{
  return misort_searchsorted_ws(dtype, sorted, n, values, m, left, out, nullptr, 0, stream);
}

// scratch of misort_unique: [sorted copy | per-block counts | scratch of the sort]
struct UniqueLayout {
  size_t off_sorted = 0, off_blk = 0, off_sort = 0, sort_bytes = 0, nblk = 0, total = 0;
};
static bool unique_layout(int dtype, size_t volume, UniqueLayout& u)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return false;
  Plan pl;
  if (make_plan(dtype, volume, volume ? volume : 1, false, false, pl) != MISORT_OK) return false;
  const size_t blk_elems = unique_block_elems(dt.bytes);
  u.nblk       = (volume + blk_elems - 1) / blk_elems;
  u.off_sorted = 0;
  u.off_blk    = align_up(volume * dt.bytes, 256);
  u.off_sort   = u.off_blk + align_up((u.nblk + 1) * sizeof(unsigned long long), 256);
  u.sort_bytes = pl.total;
  u.total      = u.off_sort + align_up(pl.total, 256) + 256;
  return true;
}

size_t misort_unique_scratch_bytes(int dtype, size_t volume)
{
  UniqueLayout u;
  return unique_layout(dtype, volume, u) ? u.total : 0;
}

int misort_unique(int dtype, const void* values_in, void* values_out, unsigned long long* count_out,
                  size_t volume, void* scratch, size_t scratch_bytes, void* stream)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return fail(MISORT_ERR_DTYPE, "unknown dtype code");
  if (!count_out) return fail(MISORT_ERR_NULL, "unique: count_out is NULL");
  if (reinterpret_cast<uintptr_t>(count_out) % 8 != 0)
    return fail(MISORT_ERR_ALIGN, "count_out not aligned to 8 bytes");
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  if (volume == 0) {
    // exactly the 8 bytes of the counter
    L.run(K_ZERO, [&] {
      hipLaunchKernelGGL(store_u64_kernel, dim3(1), dim3(1), 0, L.stream, count_out, 0ull);
    });
    return L.err == hipSuccess ? MISORT_OK : fail(MISORT_ERR_RUNTIME, hipGetErrorString(L.err));
  }
  if (!values_in || !values_out || !scratch) return fail(MISORT_ERR_NULL, "unique: NULL pointer");
  UniqueLayout u;
  if (!unique_layout(dtype, volume, u)) return fail(MISORT_ERR_UNSUPPORTED, "unique: cannot plan the sort");
  if (scratch_bytes < u.total) return fail(MISORT_ERR_SCRATCH, "unique: scratch too small");
  if (reinterpret_cast<uintptr_t>(scratch) % 256 != 0)
    return fail(MISORT_ERR_ALIGN, "scratch not aligned to 256 bytes");
  char* S      = reinterpret_cast<char*>(scratch);
  void* sorted = S + u.off_sorted;
  auto* blk    = reinterpret_cast<unsigned long long*>(S + u.off_blk);
  int rc = run_sort(L, dtype, values_in, sorted, nullptr, nullptr, volume, volume, 0, S + u.off_sort,
                    u.sort_bytes > 0 ? u.sort_bytes : 256);
  if (rc != MISORT_OK) return rc;
  const dim3 grid((unsigned)u.nblk);
#define MISORT_UNIQUE_CASE(RAW)                                                                      \
  {                                                                                                  \
    L.run(K_UNIQUE_COUNT, [&] {                                                                      \
      hipLaunchKernelGGL((unique_count_kernel<RAW>), grid, dim3(UNIQ_NT), 0, L.stream,               \
                         reinterpret_cast<const RAW*>(sorted), (uint64_t)volume, dt.xform, blk);    \
    });                                                                                              \
    L.run(K_UNIQUE_OFFSETS, [&] {                                                                    \
      hipLaunchKernelGGL(unique_offsets_kernel, dim3(1), dim3(1024), 0, L.stream, blk,               \
                         (uint64_t)u.nblk, count_out);                                               \
    });                                                                                              \
    L.run(K_UNIQUE_COMPACT, [&] {                                                                    \
      hipLaunchKernelGGL((unique_compact_kernel<RAW>), grid, dim3(UNIQ_NT), 0, L.stream,             \
                         reinterpret_cast<const RAW*>(sorted), (uint64_t)volume, dt.xform, blk,     \
                         reinterpret_cast<RAW*>(values_out));                                        \
    });                                                                                              \
  }
  switch (dt.bytes) {
    case 1: MISORT_UNIQUE_CASE(uint8_t) break;
    case 2: MISORT_UNIQUE_CASE(uint16_t) break;
    case 4: MISORT_UNIQUE_CASE(uint32_t) break;
    case 8: MISORT_UNIQUE_CASE(uint64_t) break;
    default: MISORT_UNIQUE_CASE(u128) break;
  }
#undef MISORT_UNIQUE_CASE
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

size_t misort_partition_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, int want_indices,
                                      long long kth)
{
  PartLayout u;
  if (volume == 0) return 0;
  if (partition_layout(dtype, volume, sort_dim_size, want_indices != 0, kth, u) != MISORT_OK) return 0;
  return u.total;
}

int misort_partition(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                     size_t volume, size_t sort_dim_size, long long kth, int64_t index_offset,
                     void* scratch, size_t scratch_bytes, void* stream)
{
  if (volume == 0) return MISORT_OK;
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  const bool want_indices = indices_out != nullptr;
  if (want_indices && values_out)
    return fail(MISORT_ERR_UNSUPPORTED, "partition: ask for values or for positions, not both");
  PartLayout u;
  int rc = partition_layout(dtype, volume, sort_dim_size, want_indices, kth, u);
  if (rc != MISORT_OK) return rc;
  if (!u.select)  // short rows, 1- and 2-byte values, kth out of range: the sort is the partition
    return run_sort(L, dtype, values_in, values_out, nullptr, indices_out, volume, sort_dim_size,
                    index_offset, scratch, scratch_bytes);
  if (!values_in || (!values_out && !indices_out) || !scratch)
    return fail(MISORT_ERR_NULL, "partition: NULL pointer");
  if (scratch_bytes < u.total) return fail(MISORT_ERR_SCRATCH, "partition: scratch too small");
  const size_t eb = u.pl.dt.bytes;
  auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (misaligned(values_in, eb) || (values_out && misaligned(values_out, eb)) ||
      (indices_out && misaligned(indices_out, 8)) || misaligned(scratch, 256))
    return fail(MISORT_ERR_ALIGN, "partition: misaligned pointer");
  char* S = reinterpret_cast<char*>(scratch);
  {
    auto overlaps = [&](const void* p, size_t bytes) {
      if (!p) return false;
      const char* b = reinterpret_cast<const char*>(p);
      return b < S + u.total && S < b + bytes;
    };
    if (overlaps(values_in, volume * eb) || overlaps(values_out, volume * eb) ||
        overlaps(indices_out, volume * 8))
      return fail(MISORT_ERR_ALIAS, "scratch overlaps an input or output buffer");
  }
  const bool inplace = values_out == values_in;
  void* vals         = want_indices ? nullptr : (inplace ? static_cast<void*>(S + u.off_stage) : values_out);
#define MISORT_PART_CASE(KEY) partition_select_rows<KEY>(L, u, values_in, vals, indices_out, kth, index_offset, S)
  switch (eb) {
    case 1: MISORT_PART_CASE(uint8_t); break;
    case 2: MISORT_PART_CASE(uint16_t); break;
    case 4: MISORT_PART_CASE(uint32_t); break;
    case 8: MISORT_PART_CASE(uint64_t); break;
    default: MISORT_PART_CASE(u128); break;
  }
#undef MISORT_PART_CASE
  if (!want_indices && inplace) launch_copy(L, K_COPY, values_out, S + u.off_stage, volume * eb);
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

// does misort_select serve this case?  (rows long enough for the radix path, 4- and 8-byte
// real element types, kth inside the row)
static bool select_served(const PartLayout& u) { return u.select && u.pl.dt.bytes >= 4 && u.pl.dt.xform != XF_COMPLEX; }

size_t misort_select_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, long long kth)
{
  PartLayout u;
  if (volume == 0) return 0;
  if (partition_layout(dtype, volume, sort_dim_size, false, kth, u, true) != MISORT_OK) return 0;
  return select_served(u) ? u.total : 0;
}

int misort_select(int dtype, const void* values_in, size_t volume, size_t sort_dim_size, long long kth,
                  void* kth_out, void* next_out, void* max_out, void* scratch, size_t scratch_bytes,
                  void* stream)
{
  if (volume == 0) return MISORT_OK;
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  PartLayout u;
  int rc = partition_layout(dtype, volume, sort_dim_size, false, kth, u, true);
  if (rc != MISORT_OK) return rc;
  if (!select_served(u))
    return fail(MISORT_ERR_UNSUPPORTED,
                "select: serves 4- and 8-byte real element types, rows long enough for the radix "
                "path and kth inside the row; sort instead");
  if (next_out && (unsigned long long)kth + 1 >= u.pl.row_len)
    return fail(MISORT_ERR_UNSUPPORTED, "select: no element follows kth in the row");
  if (!values_in || !scratch || (!kth_out && !next_out && !max_out))
    return fail(MISORT_ERR_NULL, "select: NULL pointer");
  if (scratch_bytes < u.total) return fail(MISORT_ERR_SCRATCH, "select: scratch too small");
  const size_t eb = u.pl.dt.bytes;
  auto misaligned = [](const void* p, size_t a) { return p && (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (misaligned(values_in, eb) || misaligned(kth_out, eb) || misaligned(next_out, eb) ||
      misaligned(max_out, eb) || misaligned(scratch, 256))
    return fail(MISORT_ERR_ALIGN, "select: misaligned pointer");
  char* S = reinterpret_cast<char*>(scratch);
  auto overlaps = [&](const void* p, size_t bytes) {
    if (!p) return false;
    const char* b = reinterpret_cast<const char*>(p);
    return b < S + u.total && S < b + bytes;
  };
  if (overlaps(values_in, volume * eb) || overlaps(kth_out, u.pl.rows * eb) ||
      overlaps(next_out, u.pl.rows * eb) || overlaps(max_out, u.pl.rows * eb))
    return fail(MISORT_ERR_ALIAS, "scratch overlaps an input or output buffer");
  if (eb == 4) select_rows<uint32_t>(L, u, values_in, kth, kth_out, next_out, max_out, S);
  else select_rows<uint64_t>(L, u, values_in, kth, kth_out, next_out, max_out, S);
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

int misort_sort_axis(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                     size_t outer, size_t k, size_t inner, int64_t index_offset, void* stream)
{
  DtypeInfo dt;
  if (!dtype_info(dtype, dt)) return fail(MISORT_ERR_DTYPE, "unknown dtype code");
  if (outer == 0 || k == 0 || inner == 0) return MISORT_OK;
  if (!values_in || (!values_out && !indices_out)) return fail(MISORT_ERR_NULL, "sort_axis: NULL pointer");
  if (values_out && indices_out)
    return fail(MISORT_ERR_UNSUPPORTED, "sort_axis: ask for values or for positions, not both");
  if (dt.bytes > 8) return fail(MISORT_ERR_UNSUPPORTED, "sort_axis: 16-byte elements take the transposed route");
  auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (misaligned(values_in, dt.bytes) || (values_out && misaligned(values_out, dt.bytes)) ||
      (indices_out && misaligned(indices_out, 8)))
    return fail(MISORT_ERR_ALIGN, "sort_axis: pointer not aligned to its element size");
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  ColParams cp;
  cp.in           = values_in;
  cp.vout         = values_out;
  cp.iout         = indices_out;
  cp.outer        = outer;
  cp.inner        = inner;
  cp.k            = (uint32_t)(k > 0xFFFFFFFFull ? 0xFFFFFFFFull : k);
  cp.index_offset = index_offset;
  cp.xform        = dt.xform;
  const bool with_idx = indices_out != nullptr || dt.xform == XF_COMPLEX;
  const bool fixf     = !with_idx && dt.xform == XF_FLOAT;
  bool served = false;
  served = launch_colsort(L, K_COLSORT, dt.bytes, cp, with_idx, fixf);
  if (!served) return fail(MISORT_ERR_UNSUPPORTED, "sort_axis: axis too long for the column kernel");
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

int misort_selftest_lds_lane_order(unsigned int rows_per_wave, unsigned long long* checked,
                                   unsigned long long* out_of_order, void* stream)
{
  if (!checked || !out_of_order) return fail(MISORT_ERR_NULL, "selftest: NULL pointer");
  std::lock_guard<std::mutex> lock(g_probe_mutex);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  unsigned long long* counts = nullptr;
  hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&counts), HIP_SYMBOL(g_selftest_counts));
  if (e != hipSuccess) return fail(MISORT_ERR_RUNTIME, std::string("hipGetSymbolAddress: ") + hipGetErrorString(e));
  hipLaunchKernelGGL(store_u64_kernel, dim3(1), dim3(1), 0, st, counts, 0ull);
  hipLaunchKernelGGL(store_u64_kernel, dim3(1), dim3(1), 0, st, counts + 1, 0ull);
  // from all digit values distinct-ish down to every lane on one word
  const uint32_t masks[6] = {0xFFu, 0x3Fu, 0x0Fu, 0x03u, 0x01u, 0x00u};
  for (int i = 0; i < 6; ++i)
    hipLaunchKernelGGL(lds_lane_order_probe_kernel, dim3(512), dim3(1024), 0, st, rows_per_wave, masks[i],
                       0x1234567u + i, counts);
  unsigned long long h[2] = {0, 0};
  e = hipMemcpyAsync(h, counts, sizeof h, hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(e));
  *checked      = h[0];
  *out_of_order = h[1];
  return MISORT_OK;
}

int misort_swap_last(const void* in, void* out, size_t outer, size_t k, size_t mid, size_t l,
                     size_t elem_bytes, void* stream)
{
  if (outer == 0 || k == 0 || mid == 0 || l == 0) return MISORT_OK;
  if (!in || !out) return fail(MISORT_ERR_NULL, "swap_last: NULL pointer");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16)
    return fail(MISORT_ERR_DTYPE, "swap_last: element size must be 1, 2, 4, 8 or 16");
  if (k > 0x7FFFFFFFull || l > 0x7FFFFFFFull || mid > 0x7FFFFFFFull ||
      ((k + 63) / 64) * ((l + 63) / 64) > 0x7FFFFFFFull)
    return fail(MISORT_ERR_UNSUPPORTED, "swap_last: extent too large");
  Launcher L;
  L.stream = reinterpret_cast<hipStream_t>(stream);
  launch_swap_last(L, K_TRANSPOSE, in, out, outer, k, mid, l, elem_bytes);
  if (L.err != hipSuccess)
    return fail(MISORT_ERR_RUNTIME, std::string("HIP error: ") + hipGetErrorString(L.err));
  return MISORT_OK;
}

}  // extern "C"
