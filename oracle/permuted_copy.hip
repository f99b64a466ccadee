// What a copy that writes whole pieces of G bytes at permuted places reaches on this GPU: the
// ceiling of any scatter pass of a radix sort, which reads its input in order and writes it in
// 128-byte lines all over the output.  A comparison figure for the roofline discussion of
// bench.py's numbers, nothing more.  Measurement infrastructure only: never linked into or
// loaded by the product.
//
// usage: permuted_copy [GiB, default 4]        prints one line per piece size
// Every workgroup reads a contiguous range; piece i of the input goes to piece pi(i) of the
// output, pi a fixed bijection of the piece numbers (multiplication by an odd constant modulo
// the power-of-two piece count, then a bit rotation), consecutive lanes to consecutive
// 16-byte units of a piece.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                      \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
      std::exit(1);                                                                   \
    }                                                                                 \
  } while (0)

template <int PIECE16>  // piece size in 16-byte units
__global__ void __launch_bounds__(1024)
permuted_copy(const uint4* __restrict__ in, uint4* __restrict__ out, size_t n16, uint64_t mult, int rot)
{
  const size_t per_wg  = n16 / gridDim.x;
  const size_t b0      = per_wg * blockIdx.x;
  const size_t npieces = n16 / PIECE16;  // a power of two
  const int bits       = 63 - __builtin_clzll(npieces);
  for (size_t i = threadIdx.x; i < per_wg; i += 1024) {
    const size_t u     = b0 + i;
    const size_t piece = u / PIECE16, within = u % PIECE16;
    size_t q = (piece * mult) & (npieces - 1);
    q        = ((q >> rot) | (q << (bits - rot))) & (npieces - 1);
    out[q * PIECE16 + within] = in[u];
  }
}

int main(int argc, char** argv)
{
  const size_t gib = argc > 1 ? (size_t)std::atoi(argv[1]) : 4;
  if (gib < 1 || gib > 32 || (gib & (gib - 1)) != 0) {
    std::fprintf(stderr, "usage: permuted_copy [GiB: 1, 2, 4, 8, 16 or 32]\n");
    return 2;
  }
  const size_t bytes = gib << 30, n16 = bytes / 16;
  uint4 *in, *out;
  CHECK(hipMalloc(&in, bytes));
  CHECK(hipMalloc(&out, bytes));
  CHECK(hipMemset(in, 1, bytes));
  CHECK(hipMemset(out, 0, bytes));
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  auto run = [&](const char* name, auto kern, uint64_t mult) {
    float best = 1e9f;
    for (int r = 0; r < 5; ++r) {
      CHECK(hipEventRecord(a, 0));
      hipLaunchKernelGGL(kern, dim3(512), dim3(1024), 0, 0, in, out, n16, mult, 7);
      CHECK(hipEventRecord(b, 0));
      CHECK(hipEventSynchronize(b));
      float ms;
      CHECK(hipEventElapsedTime(&ms, a, b));
      if (ms < best) best = ms;
    }
    std::printf("%-32s %8.3f ms  %6.2f TB/s (read + write)\n", name, best, 2.0 * bytes / best / 1e9);
    std::fflush(stdout);
  };
  const uint64_t odd = 0x9E3779B97F4A7C15ull | 1;
  run("in order (pieces of 128 B)", permuted_copy<8>, 1);
  run("permuted pieces of   64 B", permuted_copy<4>, odd);
  run("permuted pieces of  128 B", permuted_copy<8>, odd);
  run("permuted pieces of  256 B", permuted_copy<16>, odd);
  run("permuted pieces of  512 B", permuted_copy<32>, odd);
  run("permuted pieces of 1024 B", permuted_copy<64>, odd);
  run("permuted pieces of 4096 B", permuted_copy<256>, odd);
  return 0;
}
