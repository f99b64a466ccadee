// Self test of the one hardware behaviour the radix downsweep leans on without the ISA
// manual promising it: when several lanes of ONE ds_add_rtn_u32 instruction hit the same
// LDS word, gfx950 serves them in ascending lane order, so the value a lane gets back counts
// exactly the lower lanes with the same address.  The probe draws digit values with many
// equal ones per wavefront (digit_mask picks how many distinct values), ranks every lane
// both ways - returning add and the 8-ballot match - with 16 wavefronts per workgroup
// working on the LDS at once, and counts the lanes where the two disagree.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace misort {

__device__ unsigned long long g_selftest_counts[2];  // {lanes checked, lanes out of order}

__global__ void __launch_bounds__(1024)
lds_lane_order_probe_kernel(uint32_t rows_per_wave, uint32_t digit_mask, uint32_t seed,
                            unsigned long long* counts)
{
  __shared__ uint32_t ctr[16 * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t* my   = ctr + wave * 256;
  for (int i = lane; i < 256; i += 64) my[i] = 0;
  __syncthreads();
  unsigned long long bad = 0, cnt = 0;
  uint32_t x = seed ^ (blockIdx.x * 0x9E3779B9u) ^ (threadIdx.x * 0x85EBCA6Bu);
  for (uint32_t r = 0; r < rows_per_wave; ++r) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    const uint32_t d   = (x >> 11) & digit_mask & 255u;
    const uint32_t old = atomicAdd(&my[d], 1u);
    uint64_t peers     = ~0ull;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const bool bit    = (d >> b) & 1u;
      const uint64_t bl = __ballot(bit);
      peers &= bit ? bl : ~bl;
    }
    const uint32_t below = __popcll(peers & ((1ull << lane) - 1ull));
    const uint32_t k     = __popcll(peers);
    const uint32_t after = __hip_atomic_load(&my[d], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    // the wave-row added k to the counter, which stood at after - k before it
    bad += old != after - k + below;
    ++cnt;
  }
  atomicAdd(&counts[0], cnt);
  atomicAdd(&counts[1], bad);
}

}  // namespace misort
