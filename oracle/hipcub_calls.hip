// What the reference's GPU sort path reaches on this GPU when its CUB calls are served by
// hipCUB (rocPRIM back-end): a comparison baseline for bench.py's figures, nothing more.
// Measurement infrastructure only: never linked into or loaded by the product.
//
// It restates, for 1-D input, the sequence of device work that the reference enqueues:
//   argsort (src/cunumeric/sort/sort.cu:1694-1751, then src/cunumeric/sort/cub_sort.cuh:111-147):
//     fill the int64 index output with 0..n-1, copy it (the indices are sorted "in place", so
//     CUB gets a copy as its input), DeviceRadixSort::SortPairs over the full key width;
//   sort (cub_sort.cuh:55-71): DeviceRadixSort::SortKeys over the full key width.
// The sizing calls and the allocations of the reference (a memory pool there) are made once,
// outside the timed region, which favours the baseline.
//
// usage: hipcub_calls <c1|c2|c4|i64small> [log2 n] [repetitions]     prints one JSON line
//   c1: sort of int32, uniform          c2: stable argsort of float32, N(0,1) with 1 % NaN,
//   c4: stable argsort of int64, 16 distinct values with Zipf(1.2) weights   and 1 % zeros
//   i64small: stable argsort of int64 values below 50000
#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CHECK(x)                                                                        \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_));   \
      std::exit(1);                                                                     \
    }                                                                                   \
  } while (0)

__device__ inline uint64_t mix(uint64_t x)
{
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

__global__ void gen_i32(int32_t* out, size_t n)
{
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = (int32_t)mix(i);
}

__global__ void gen_f32(float* out, size_t n)
{
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const uint64_t h = mix(i), g = mix(h);
    const float u1 = ((h >> 40) + 1) * (1.0f / 16777217.0f), u2 = (g >> 40) * (1.0f / 16777216.0f);
    float v        = sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
    const uint32_t s = (uint32_t)(g & 0xFFFF);
    if (s < 655) v = __builtin_nanf("");
    else if (s < 983) v = -0.0f;
    else if (s < 1311) v = 0.0f;
    out[i] = v;
  }
}

__global__ void gen_zipf16(int64_t* out, size_t n, const int64_t* values, const float* cdf)
{
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const float u = (mix(i) >> 40) * (1.0f / 16777216.0f);
    int k         = 0;
    while (k < 15 && u >= cdf[k]) ++k;
    out[i] = values[k];
  }
}

__global__ void gen_small_i64(int64_t* out, size_t n, uint64_t range)
{
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = (int64_t)(mix(i) % range);
}

__global__ void iota_i64(int64_t* out, size_t n)
{
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = (int64_t)i;
}

template <typename K>
static double run(const char* name, const K* keys_in, size_t n, bool argsort, int reps)
{
  K* keys_out       = nullptr;
  int64_t *idx_out = nullptr, *idx_in = nullptr;
  void* temp        = nullptr;
  size_t temp_bytes = 0;
  CHECK(hipMalloc(&keys_out, n * sizeof(K)));
  if (argsort) {
    CHECK(hipMalloc(&idx_out, n * 8));
    CHECK(hipMalloc(&idx_in, n * 8));
    CHECK(hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, keys_in, keys_out, idx_in, idx_out, n, 0,
                                             (int)sizeof(K) * 8, 0));
  } else {
    CHECK(hipcub::DeviceRadixSort::SortKeys(nullptr, temp_bytes, keys_in, keys_out, n, 0, (int)sizeof(K) * 8, 0));
  }
  CHECK(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
  auto once = [&] {
    if (argsort) {
      hipLaunchKernelGGL(iota_i64, dim3(4096), dim3(256), 0, 0, idx_out, n);
      CHECK(hipMemcpyAsync(idx_in, idx_out, n * 8, hipMemcpyDeviceToDevice, 0));
      CHECK(hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys_in, keys_out, idx_in, idx_out, n, 0,
                                               (int)sizeof(K) * 8, 0));
    } else {
      CHECK(hipcub::DeviceRadixSort::SortKeys(temp, temp_bytes, keys_in, keys_out, n, 0, (int)sizeof(K) * 8, 0));
    }
  };
  once();
  once();
  CHECK(hipDeviceSynchronize());
  std::vector<float> ms(reps);
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  for (int r = 0; r < reps; ++r) {
    CHECK(hipEventRecord(a, 0));
    once();
    CHECK(hipEventRecord(b, 0));
    CHECK(hipEventSynchronize(b));
    CHECK(hipEventElapsedTime(&ms[r], a, b));
  }
  std::sort(ms.begin(), ms.end());
  const double med = ms[reps / 2];
  // the sort alone, without the index fill and copy
  std::vector<float> ms2(reps);
  for (int r = 0; r < reps; ++r) {
    CHECK(hipEventRecord(a, 0));
    if (argsort)
      CHECK(hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys_in, keys_out, idx_in, idx_out, n, 0,
                                               (int)sizeof(K) * 8, 0));
    else
      CHECK(hipcub::DeviceRadixSort::SortKeys(temp, temp_bytes, keys_in, keys_out, n, 0, (int)sizeof(K) * 8, 0));
    CHECK(hipEventRecord(b, 0));
    CHECK(hipEventSynchronize(b));
    CHECK(hipEventElapsedTime(&ms2[r], a, b));
  }
  std::sort(ms2.begin(), ms2.end());
  // a look at the result: the first 2^20 keys of the output must be non-decreasing (NaN last)
  const size_t m = std::min<size_t>(n, 1u << 20);
  std::vector<K> h(m);
  CHECK(hipMemcpy(h.data(), keys_out, m * sizeof(K), hipMemcpyDeviceToHost));
  bool ok = true;
  for (size_t i = 1; i < m; ++i) ok = ok && !(h[i] < h[i - 1]);
  std::printf(
    "{\"baseline\": \"hipcub\", \"workload\": \"%s\", \"n\": %zu, \"argsort\": %s, \"ms_median\": %.4f, "
    "\"Gkeys_per_s\": %.2f, \"library_call_only_ms\": %.4f, \"temp_bytes\": %zu, \"calls\": %d, "
    "\"head_sorted\": %s}\n",
    name, n, argsort ? "true" : "false", med, n / med / 1e6, (double)ms2[reps / 2], temp_bytes, reps,
    ok ? "true" : "false");
  CHECK(hipFree(temp));
  CHECK(hipFree(keys_out));
  if (idx_out) CHECK(hipFree(idx_out));
  if (idx_in) CHECK(hipFree(idx_in));
  return med;
}

int main(int argc, char** argv)
{
  const char* w  = argc > 1 ? argv[1] : "c2";
  const int lg   = argc > 2 ? std::atoi(argv[2]) : (std::strcmp(w, "c1") == 0 ? 24 : 28);
  const int reps = argc > 3 ? std::atoi(argv[3]) : 10;
  if (lg < 1 || lg > 30 || reps < 1) {
    std::fprintf(stderr, "usage: hipcub_calls <c1|c2|c4|i64small> [log2 n <= 30] [repetitions]\n");
    return 2;
  }
  const size_t n = (size_t)1 << lg;
  if (std::strcmp(w, "c1") == 0) {
    int32_t* k;
    CHECK(hipMalloc(&k, n * 4));
    hipLaunchKernelGGL(gen_i32, dim3(4096), dim3(256), 0, 0, k, n);
    run<int32_t>(w, k, n, false, reps);
  } else if (std::strcmp(w, "c2") == 0) {
    float* k;
    CHECK(hipMalloc(&k, n * 4));
    hipLaunchKernelGGL(gen_f32, dim3(4096), dim3(256), 0, 0, k, n);
    run<float>(w, k, n, true, reps);
  } else if (std::strcmp(w, "c4") == 0) {
    int64_t hv[16];
    float hc[16];
    double tot = 0, acc = 0;
    for (int i = 0; i < 16; ++i) tot += std::pow(i + 1.0, -1.2);
    uint64_t s = 4;
    for (int i = 0; i < 16; ++i) {
      s     = s * 6364136223846793005ull + 1442695040888963407ull;
      hv[i] = (int64_t)(s ^ (s >> 29));
      acc += std::pow(i + 1.0, -1.2) / tot;
      hc[i] = (float)acc;
    }
    int64_t *k, *dv;
    float* dc;
    CHECK(hipMalloc(&k, n * 8));
    CHECK(hipMalloc(&dv, sizeof hv));
    CHECK(hipMalloc(&dc, sizeof hc));
    CHECK(hipMemcpy(dv, hv, sizeof hv, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(dc, hc, sizeof hc, hipMemcpyHostToDevice));
    hipLaunchKernelGGL(gen_zipf16, dim3(4096), dim3(256), 0, 0, k, n, dv, dc);
    run<int64_t>(w, k, n, true, reps);
  } else if (std::strcmp(w, "i64small") == 0) {
    int64_t* k;
    CHECK(hipMalloc(&k, n * 8));
    hipLaunchKernelGGL(gen_small_i64, dim3(4096), dim3(256), 0, 0, k, n, (uint64_t)50000);
    run<int64_t>(w, k, n, true, reps);
  } else {
    std::fprintf(stderr, "unknown workload %s\n", w);
    return 2;
  }
  return 0;
}
