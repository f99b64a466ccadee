/*
 * misort -- C ABI of the MI355X (gfx950) local sort.
 *
 * This is the seam a cuNumeric build would bind in place of its per-dtype
 * `cub_local_sort` / `thrust_local_sort` overloads, i.e. the body of
 *   local_sort<CODE>(values_in, values_out, indices_in, indices_out,
 *                    volume, sort_dim_size, stable, stream)
 * (reference: src/cunumeric/sort/sort.cu:52-85, typed declarations at
 * src/cunumeric/sort/cub_sort.h:21-115 and src/cunumeric/sort/thrust_sort.h:21-145).
 *
 * Plain pointers and sizes only.  All pointers are device pointers of the GPU
 * that is current on the calling thread.  All work is enqueued on `stream`;
 * no entry point synchronises the host with the device (except the *_profiled
 * variant, which is a measurement aid) and none allocates device memory.
 */
#ifndef MISORT_H_
#define MISORT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element type codes, in the order of cuNumeric's SUPPORTED_DTYPES table (reference:
 * cunumeric/utils.py:29-44).  They are this library's own numbers: a binding maps its
 * framework's type enumeration to them by name (a switch over the framework's enumerators
 * that returns MISORT_<NAME>), never by casting one enumeration to the other. */
typedef enum misort_dtype {
  MISORT_BOOL       = 0,
  MISORT_INT8       = 1,
  MISORT_INT16      = 2,
  MISORT_INT32      = 3,
  MISORT_INT64      = 4,
  MISORT_UINT8      = 5,
  MISORT_UINT16     = 6,
  MISORT_UINT32     = 7,
  MISORT_UINT64     = 8,
  MISORT_FLOAT16    = 9,
  MISORT_FLOAT32    = 10,
  MISORT_FLOAT64    = 11,
  MISORT_COMPLEX64  = 12,
  MISORT_COMPLEX128 = 13
} misort_dtype;

/* Status codes.  The reference aborts on any CUDA error (CHECK_CUDA,
 * src/cunumeric/cuda_help.h:62-66); this library returns a code instead and
 * never aborts. */
typedef enum misort_status {
  MISORT_OK                 = 0,
  MISORT_ERR_DTYPE          = 1, /* dtype code not one of misort_dtype            */
  MISORT_ERR_NULL           = 2, /* a required pointer is NULL                    */
  MISORT_ERR_SHAPE          = 3, /* volume is not a multiple of sort_dim_size     */
  MISORT_ERR_SCRATCH        = 4, /* scratch_bytes smaller than misort_scratch_bytes */
  MISORT_ERR_ALIGN          = 5, /* a pointer is not aligned to its element size / scratch not 256-B aligned */
  MISORT_ERR_RUNTIME        = 6, /* a HIP call failed; see misort_last_error()    */
  MISORT_ERR_ALIAS          = 7, /* output overlaps scratch                        */
  MISORT_ERR_UNSUPPORTED    = 8  /* a size beyond what the kernels index          */
} misort_status;

/* Library version: major*10000 + minor*100 + patch. */
int misort_version(void);

/* Size in bytes of one element of `dtype`, or 0 for an unknown code. */
size_t misort_dtype_size(int dtype);

/* Text of the last error raised on the calling thread ("" if none). */
const char* misort_last_error(void);

/*
 * Scratch the caller must provide to misort_local for the same arguments.
 * `argsort` != 0 means indices_out will be non-NULL; `has_indices_in` != 0
 * means indices_in will be non-NULL (a caller-filled int64 payload).
 * Replaces the null-pointer dry run the reference uses to size CUB's temporary
 * storage (src/cunumeric/sort/cub_sort.cuh:60-62) and the key / index staging
 * buffers it allocates from the Legate pool (cub_sort.cuh:46-52, 110-116;
 * sort.cu:1698).  Returns 0 when volume == 0.
 * The radix path of 4-byte and wider keys includes one byte per element for a digit
 * side-band (each pass can leave the next pass's digit of every key there, so that the next
 * count reads bytes instead of keys); MISORT_SIDE_BAND=0 in the environment before the first
 * call into the library leaves it out (give the query and the sort the same environment).
 * Radix passes over a digit that is the same in every key are skipped (decided on the device,
 * nothing is read back); MISORT_SKIP_PASSES=0 runs them all.  Sorts of 256 MB of keys and
 * more also leave out the passes over constant most significant digits (the last pass whose
 * digit varies writes the result); MISORT_EARLY_LAST_BYTES=<bytes> moves that limit.  All
 * four variables are read once, when the library is first used.
 */
size_t misort_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                            int has_indices_in);

/*
 * Sort `volume / sort_dim_size` independent, contiguous rows of
 * `sort_dim_size` elements each, ascending, NumPy ordering (NaN last, -0 == +0,
 * complex lexicographic).  Always stable, whatever `stable` says.
 *
 *   indices_out == NULL : keys only; sorted rows are written to values_out
 *                         (values_out == values_in is allowed).
 *   indices_out != NULL : argsort; indices_out receives, per row, the payload
 *                         carried with each key.  With indices_in == NULL the
 *                         payload is the element's position within its row
 *                         plus `index_offset` (what the reference pre-fills
 *                         with thrust::sequence / modulusWithOffset,
 *                         sort.cu:1713-1725).  With indices_in != NULL the
 *                         caller's int64 payload is carried instead
 *                         (indices_in == indices_out is allowed).  values_out
 *                         may be NULL (the reference discards the sorted key
 *                         copy of an argsort, sort.cu:1800-1803); if non-NULL
 *                         it receives the sorted keys.
 *
 * Reference interface replaced: local_sort<CODE>, src/cunumeric/sort/sort.cu:52-85.
 */
int misort_local(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                 int64_t* indices_out, size_t volume, size_t sort_dim_size, int stable,
                 int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream);

/*
 * Measurement aid: same as misort_local, but brackets every kernel launch with
 * HIP events on `stream`, synchronises, and reports the launches.
 * On return *n_kernels is the number of launches; for i < min(*n_kernels, max_kernels)
 * kernel_ms[i] is the duration in milliseconds and kernel_ids[i] the kernel
 * kind (see misort_kernel_name).  No counterpart in the reference.
 */
int misort_local_profiled(int dtype, const void* values_in, void* values_out,
                          const int64_t* indices_in, int64_t* indices_out, size_t volume,
                          size_t sort_dim_size, int stable, int64_t index_offset, void* scratch,
                          size_t scratch_bytes, void* stream, float* kernel_ms, int* kernel_ids,
                          int max_kernels, int* n_kernels);

/* Name of a kernel kind reported by misort_local_profiled ("" if unknown). */
const char* misort_kernel_name(int kernel_id);

/*
 * Description of the plan misort_local would execute: number of radix passes,
 * digit width, tile size, which row strategy.  Written as a short text into
 * buf (NUL-terminated, truncated to buf_bytes).  Returns MISORT_OK or an error.
 */
int misort_describe_plan(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                         int has_indices_in, char* buf, size_t buf_bytes);

/*
 * Insertion indices into a sorted 1-D array (first of the "next" steps after the sort):
 *   left != 0: out[j] = number of elements of sorted[] that order before values[j]
 *   left == 0: out[j] = number of elements that do not order after values[j]
 * under the order the sorts of this library produce (NumPy's).  sorted[] has n elements
 * and values[] m, both of dtype `dtype`; out[] has m int64.  Replaces the SEARCHSORTED
 * task body for one GPU (reference: src/cunumeric/sort/searchsorted.cu:25-110; the
 * Python side is cunumeric/array.py:3637-3709, cunumeric/deferred.py:3511-3533).
 */
int misort_searchsorted(int dtype, const void* sorted, size_t n, const void* values, size_t m,
                        int left, int64_t* out, void* stream);

/*
 * misort_searchsorted with a workspace.  Many random queries into an array far larger than
 * the caches spend their time fetching one cache line per probe; with a workspace the queries
 * are sorted first (by this library, with their positions), so that neighbouring threads
 * probe neighbouring elements, and every answer is stored at the position its query came
 * from.  misort_searchsorted_scratch_bytes returns 0 where that does not pay (few queries or
 * a small array); scratch may then be NULL and the call is misort_searchsorted.  No
 * counterpart in the reference (one cub::LowerBound / UpperBound per query,
 * src/cunumeric/sort/searchsorted.cu:25-63).
 */
size_t misort_searchsorted_scratch_bytes(int dtype, size_t n, size_t m);
int misort_searchsorted_ws(int dtype, const void* sorted, size_t n, const void* values, size_t m,
                           int left, int64_t* out, void* scratch, size_t scratch_bytes, void* stream);

/*
 * Sorted distinct elements of an array of `volume` elements (any shape: it is treated as
 * flat).  values_out must have room for `volume` elements; the number written goes to
 * *count_out (device memory, 8-byte aligned), which the caller reads after synchronising
 * the stream.  -0 and +0 are one value; all NaNs (complex: every element with a NaN part)
 * are one value.  Scratch as for misort_local, sized by misort_unique_scratch_bytes.
 * Replaces the UNIQUE task body for one GPU (reference: src/cunumeric/set/unique.cu:150-180,
 * thrust::sort + thrust::unique; Python side cunumeric/module.py:6800-6874,
 * cunumeric/deferred.py:3490-3508).
 */
size_t misort_unique_scratch_bytes(int dtype, size_t volume);
int misort_unique(int dtype, const void* values_in, void* values_out, unsigned long long* count_out,
                  size_t volume, void* scratch, size_t scratch_bytes, void* stream);

/*
 * Partition every row around the element a sort would leave at position kth (0 <= kth <
 * sort_dim_size): afterwards that element is at kth, nothing that orders after it stands
 * before it and nothing that orders before it stands after it (NumPy's partition /
 * argpartition contract; equal elements keep their input order).  Give values_out for the
 * partitioned elements or indices_out for their positions within the row (+ index_offset),
 * not both.  values_out may be values_in.  Long rows of 4-byte and wider elements are
 * partitioned by selection (one histogram pass per key byte to find the pivot, then one
 * three-way split pass); everything else, and a kth outside the row, runs the ordinary
 * sort, which is a valid partition.  The reference sorts in every case
 * (cunumeric/deferred.py:3559-3578 calls sort_task; src/cunumeric/sort/sort.cu:52-85).
 */
size_t misort_partition_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, int want_indices,
                                      long long kth);
int misort_partition(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                     size_t volume, size_t sort_dim_size, long long kth, int64_t index_offset,
                     void* scratch, size_t scratch_bytes, void* stream);

/*
 * The selection alone, for callers that want order statistics and not a partitioned row
 * (quantile / percentile: cunumeric/module.py:8248-8531 sorts the whole array and reads
 * two elements per quantile; src/cunumeric/sort/sort.cu:52-85 is that sort).  Per row of
 * sort_dim_size elements: kth_out[row] = the element a sort would leave at position kth,
 * next_out[row] = the one at kth + 1 (kth + 1 must lie inside the row), max_out[row] = the
 * last element in sort order (NaN for a floating-point row that holds a NaN).  Each of the
 * three may be NULL; each has volume / sort_dim_size elements of the element type.  The row
 * is read, not written.  Floating-point results come back as the keys keep them: a zero as
 * +0, a NaN as the default quiet NaN.  Served: 4- and 8-byte integer and floating-point
 * types on rows long enough for the radix path with 0 <= kth < sort_dim_size; otherwise
 * misort_select_scratch_bytes returns 0 and misort_select MISORT_ERR_UNSUPPORTED (sort
 * instead).  Work: one read of the row per leading key byte until the keys that still match
 * are few (two reads when the leading bytes vary), and one more for next_out only when those
 * keys hold nothing above the kth key; against four to eight scattered passes of a sort.
 */
size_t misort_select_scratch_bytes(int dtype, size_t volume, size_t sort_dim_size, long long kth);
int misort_select(int dtype, const void* values_in, size_t volume, size_t sort_dim_size, long long kth,
                  void* kth_out, void* next_out, void* max_out, void* scratch, size_t scratch_bytes,
                  void* stream);

/*
 * Sort a dense (outer, k, inner) array along its middle axis: every column (o, :, i) on its
 * own, result in the same layout; give values_out (may be values_in) or indices_out
 * (positions along the axis + index_offset), not both.  Served for short axes (k up to
 * 1024 for elements of at most 4 bytes, 512 for 8-byte ones; 16-byte elements not at
 * all): otherwise MISORT_ERR_UNSUPPORTED, and the caller
 * takes the transposed route (misort_swap_last + misort_local + misort_swap_last), which is
 * what the reference always does (cunumeric/sort.py:47-83).  Needs no scratch.
 */
int misort_sort_axis(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                     size_t outer, size_t k, size_t inner, int64_t index_offset, void* stream);

/*
 * misort_scratch_bytes / misort_local with the number of chunks (one workgroup each) that a
 * radix pass over the whole array is cut into given by the caller; a chunk is a run of
 * consecutive tiles that one workgroup walks in order.  target_chunks == 0 is the built-in
 * choice (two per CU), which is what the plain entry points use.  The value is part of the
 * plan: give the same one to the query and to the sort.  No counterpart in the reference
 * (CUB picks its grid itself, src/cunumeric/sort/cub_sort.cuh:60-71); for callers that
 * share the GPU between several streams, and for tests of the multi-tile loop on small arrays.
 */
size_t misort_scratch_bytes_chunked(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                                    int has_indices_in, size_t target_chunks);
int misort_local_chunked(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                         int64_t* indices_out, size_t volume, size_t sort_dim_size, int stable,
                         int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream,
                         size_t target_chunks);

/*
 * misort_scratch_bytes / misort_local with choices that are otherwise built in, per call (a
 * NULL pointer, or a zeroed struct with early_last_min_bytes = bucket_path = low_cardinality
 * = -1, means "as misort_local").  No counterpart in the reference; for tests that have to reach the code for
 * large or unusual inputs with small arrays, and for measurements.  Give the query and the
 * sort the same options.
 *   target_chunks         as misort_local_chunked (0: built in)
 *   early_last_min_bytes  from how many bytes of keys on the passes over constant most
 *                         significant digits are left out as well (< 0: built in, 256 MB)
 *   bucket_path           rows of up to about two million elements (all rows of the call
 *                         together) are sorted in four launches (splitters from a sorted sample,
 *                         count, scatter into at most 256 bins, radix sort of every bin inside
 *                         one workgroup) instead of two launches per digit.  < 0: built in (2-
 *                         to 8-byte elements, up to the lengths where the radix passes catch
 *                         up); 0: never; > 0: for all rows of 1- to 8-byte elements, whatever
 *                         their length
 *   bucket_bins           number of bins, 2 .. 256 (0: built in, one per 1024 elements)
 *   bucket_cap            longest bin that is sorted in registers; longer ones take the
 *                         workgroup's loop through global memory (0: built in, 16384)
 *   bucket_oversample     sample keys drawn per bin, 1 .. 32 (0: built in: 16, and 32 for rows
 *                         whose bins average more than 5/12 of bucket_cap; fewer samples
 *                         give uneven bins: tests of bins that outgrow the registers)
 *   low_cardinality       single rows too long for that path, 4- and 8-byte keys, outputs apart
 *                         from the inputs: the path is tried all the same where a sample of the
 *                         row holds at most 255 distinct keys (each of them then gets a bin of
 *                         its own, which needs no sorting), and the radix kernels return at once
 *                         if it went through; decided on the device, nothing is read back.
 *                         < 0: built in (rows of 2^27 elements and more: the attempt costs
 *                         35-50 us where it is called off); 0: never; 1: rows of any length;
 *                         2: tried with any sample (tests of the way back to the radix path)
 *   counting_sort         values-only sorts of one row of 2-byte elements are counted (65536
 *                         counters) instead of radix-sorted.  < 0: built in (from 2^24 float16
 *                         and 2^26 integer elements on, where counting is ahead); 0: never;
 *                         > 0: every such row that is too long for the row kernels
 *   upper_first           long sorts of 8-byte keys (outputs apart from the inputs) run their
 *                         radix passes over the upper five bytes only, and one read of the
 *                         result then sorts the short runs of keys that agree in those; a
 *                         sample of the keys decides whether that is tried, and the eight
 *                         passes follow on the device if a run was too long to sort that way.
 *                         < 0: built in (from 2^25 elements on); 0: never; 1: any length;
 *                         2: tried whatever the sample says (tests of the way back)
 */
typedef struct misort_options {
  size_t target_chunks;
  long long early_last_min_bytes;
  int bucket_path;
  unsigned bucket_bins;
  unsigned bucket_cap;
  int low_cardinality;
  unsigned bucket_oversample;
  int counting_sort;
  int upper_first;
} misort_options;
size_t misort_scratch_bytes_opts(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                                 int has_indices_in, const misort_options* options);
int misort_local_opts(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                      int64_t* indices_out, size_t volume, size_t sort_dim_size, int stable,
                      int64_t index_offset, void* scratch, size_t scratch_bytes, void* stream,
                      const misort_options* options);
/* misort_describe_plan for the plan that misort_local_opts would execute with `options`. */
int misort_describe_plan_opts(int dtype, size_t volume, size_t sort_dim_size, int argsort,
                              int has_indices_in, const misort_options* options, char* buf,
                              size_t buf_bytes);

/*
 * One-time set-up for the GPU that is current on the calling thread, optional: looks up the
 * address of the library's own scratch buffer (misort_local_static) and decides how the radix
 * scatter ranks on this GPU (misort_rank_mode).  Both happen by themselves in the first call
 * that needs them; a caller that records its calls into a HIP graph, or must not see a
 * synchronisation later, calls this first, outside any capture.  No counterpart in the
 * reference (static registration, src/cunumeric/sort/sort.cc:73-81, is the nearest thing).
 */
int misort_init(void);

/*
 * How the radix scatter ranks the keys of a wavefront on the current GPU: 1 = one returning
 * LDS add per key, 2 = wave ballots, 0 = not decided yet (no sort has run here and
 * misort_init was not called).  The adds are stable only where the LDS serves the lanes of
 * one instruction that hit the same word in ascending lane order; the library uses them only
 * on gfx950 and only after a probe of 25 million lane operations on that GPU (about 0.35 ms,
 * on a stream of its own, once per GPU and process) has found every lane in order, and
 * MISORT_RANK_BALLOT=1 in the environment rules them out.  No counterpart in the reference.
 */
int misort_rank_mode(void);

/*
 * misort_local without a scratch argument and without any allocation: the scratch is a
 * buffer of MISORT_STATIC_SCRATCH_BYTES that the library itself holds in device memory on
 * every GPU it runs on, until the process ends.  No counterpart in the reference (which
 * allocates from the Legate pool in every call, src/cunumeric/sort/cub_sort.cuh:46-62); it is
 * for callers that cannot allocate: tight serving loops, harnesses that forbid hipMalloc, code
 * that records into a HIP graph (call misort_init before the capture starts: the first call
 * on a GPU looks the buffer's address up and probes the LDS, neither of which may be
 * recorded).  Same arguments and results as misort_local.  A sort
 * whose misort_scratch_bytes exceeds MISORT_STATIC_SCRATCH_BYTES is refused with
 * MISORT_ERR_SCRATCH (nothing is launched).  All calls on one GPU share the one buffer:
 * calls that overlap in time on the same GPU (different streams or threads) race; calls
 * ordered on one stream are safe.  The first call on a GPU looks the buffer's address up
 * (hipGetSymbolAddress); no call uses hipMalloc, hipFree or an allocating library routine.
 * `stream` must belong to the GPU that is current on the calling thread (each GPU has its own
 * copy of the buffer); a stream of another GPU is refused with MISORT_ERR_UNSUPPORTED.
 */
#define MISORT_STATIC_SCRATCH_BYTES (64u << 20)
int misort_local_static(int dtype, const void* values_in, void* values_out, const int64_t* indices_in,
                        int64_t* indices_out, size_t volume, size_t sort_dim_size, int stable,
                        int64_t index_offset, void* stream);

/*
 * Self test, no counterpart in the reference.  The radix scatter ranks the keys of a
 * wavefront with one returning LDS add per key, which is stable only because gfx950 serves
 * the lanes of one such instruction that hit the same word in ascending lane order.  This
 * call checks exactly that on the current GPU: 6 x 512 workgroups x 16 wavefronts x
 * rows_per_wave instructions with few distinct addresses, every lane compared with its rank
 * by the ballot match.  *checked receives the number of lanes compared, *out_of_order the
 * number that disagreed (0 on every MI355X seen).  Host pointers; synchronises `stream`.
 * The library runs a short form of the same probe by itself before it first uses the adds on a
 * GPU (misort_rank_mode); setting MISORT_RANK_BALLOT=1 in the environment before the first
 * call into the library makes every sort rank by ballots instead.
 */
int misort_selftest_lds_lane_order(unsigned int rows_per_wave, unsigned long long* checked,
                                   unsigned long long* out_of_order, void* stream);

/*
 * Dense row-major copy with one axis swapped with the last one:
 *   out[o][l][m][k] = in[o][k][m][l]   (in is outer x k x mid x l, out is outer x l x mid x k)
 * for elements of `elem_bytes` (1, 2, 4, 8 or 16) bytes.  mid == 1 is a batched 2-D
 * transpose.  This is the transposed dense copy the reference makes before sorting along a
 * non-last axis and the transposed view it returns afterwards (reference:
 * cunumeric/sort.py:47-83, `swapped_copy.copy(swapped, deep=True)`; the copy itself is the
 * UNARY_OP COPY task, cunumeric/deferred.py:392-401).  in and out must not overlap.
 */
int misort_swap_last(const void* in, void* out, size_t outer, size_t k, size_t mid, size_t l,
                     size_t elem_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MISORT_H_ */
