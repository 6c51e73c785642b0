// Helpers of the kernels that hold a whole reduction unit (a BatchNormalization
// channel, a long row) on one CU: NR vectors per thread in registers, NS more
// in LDS.
#pragma once
#include <type_traits>

#include "common.cuh"

namespace nblahip {

constexpr int kOnchipBlock = 1024;

template <int TB = kOnchipBlock>
__device__ __forceinline__ float onchip_block_sum(float v, float *red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  lds_barrier(); // earlier readers of red are done
  if ((threadIdx.x & (kWave - 1)) == 0) red[wave] = v;
  lds_barrier();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < TB / kWave; ++i) t += red[i];
  return t;
}

// The same value, opaque to the optimiser: offsets computed from it are not
// merged with those of an earlier pass (kept alive across the passes, the 25
// offsets of a thread cost 25 registers and the kernel spills).
__device__ __forceinline__ uint32_t fresh(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Hides a register-held vector from the optimiser (keep_packed does so for
// half data only): what pass 1 derived from it (x - mean, xh) is then computed
// again in pass 2 instead of being kept alive, or spilled, across the passes.
template <typename T, int VEC> __device__ __forceinline__ void forget(RawVec<T, VEC> &r) {
  if constexpr (sizeof(T) == 4) {
    asm volatile("" : "+v"(r.v.x), "+v"(r.v.y), "+v"(r.v.z), "+v"(r.v.w));
  } else {
    keep_packed<T, VEC>(r);
  }
}

// v again, but only once `after` has been computed: ties the addresses of a
// batch of loads to the previous batch's results, so the compiler cannot issue
// every batch up front (25 batches' worth of registers).
__device__ __forceinline__ uint32_t fresh_after(uint32_t v, float after) {
  asm volatile("" : "+v"(v) : "v"(after));
  return v;
}

__device__ __forceinline__ uint32_t fresh_after(uint32_t v, uint32_t after) {
  asm volatile("" : "+v"(v) : "v"(after));
  return v;
}

// LDS slot of a parked vector: 16 bytes, or 8 for half planes of 4k (not 8k)
// elements, which are read in 8-byte vectors.
template <typename T, int VEC>
using Slot = std::conditional_t<sizeof(RawVec<T, VEC>) == 16, uint4, uint2>;

} // namespace nblahip
