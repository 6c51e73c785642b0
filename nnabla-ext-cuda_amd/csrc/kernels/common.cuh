// Device-side building blocks shared by every normalization kernel:
// 128-bit vector access with fp32 conversion, wavefront-64 reductions (DPP for
// the in-row steps, lane reads for the cross-row steps), LDS block reductions
// and Welford/Chan merging.  gfx950 only: a wavefront is 64 lanes.
#pragma once

// The kernels assume the CDNA4 part they are tuned for: 64-lane waves, 160 KB of
// LDS per workgroup (the on-chip layouts declare up to 147 KB statically), 512
// vector registers per SIMD lane.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "nblahip kernels are written for gfx950 (MI355X); build with ARCH=gfx950"
#endif

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nblahip {

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Element traits: VEC elements per 16-byte access.
// ---------------------------------------------------------------------------
template <typename T> struct FullVec;
template <> struct FullVec<float> { static constexpr int value = 4; };
template <> struct FullVec<__half> { static constexpr int value = 8; };
// 8-byte vectors for half rows of 4k elements (float: the full vector again).
template <typename T> struct MidVec { static constexpr int value = 4; };

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) {
  return __half2float(v);
}
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) {
  return __float2half(v); // round to nearest even
}

// Load VEC consecutive elements starting at p (p aligned to VEC*sizeof(T))
// and widen them to float.
template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T *__restrict__ p, float (&out)[VEC]) {
  if constexpr (VEC == 1) {
    out[0] = to_f32<T>(p[0]);
  } else if constexpr (sizeof(T) == 4) {
    static_assert(VEC == 4, "float vectors are 4 wide");
    const float4 v = *reinterpret_cast<const float4 *>(p);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else if constexpr (VEC == 4) { // half, 8-byte access
    const uint2 raw = *reinterpret_cast<const uint2 *>(p);
    const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float2 f = __half22float2(h[i]);
      out[2 * i] = f.x;
      out[2 * i + 1] = f.y;
    }
  } else {
    static_assert(VEC == 8, "half vectors are 8 or 4 wide");
    const uint4 raw = *reinterpret_cast<const uint4 *>(p);
    const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 f = __half22float2(h[i]);
      out[2 * i] = f.x;
      out[2 * i + 1] = f.y;
    }
  }
}

// Vector stores of outputs are non-temporal by default: an output is written
// once and not read again by the call, so it should not displace the inputs
// (which the second pass of a split reduction reads again) from L2 and the
// Infinity Cache.  Measured on [32,256,56,56] fp32 BatchNormalization: backward
// apply 44.4 -> 41.9 us, the four kernels 125.8 -> 118.9 us.  (Non-temporal
// loads were measured too and lose: the second pass then misses the cache.)
// STREAM = false keeps the ordinary store: for kernels whose wave writes short
// pieces of many cache lines (the channel-last tiles), where neighbouring
// blocks complete the lines in L2; non-temporal stores of such pieces cost 3x.
typedef float native_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t native_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t native_u2 __attribute__((ext_vector_type(2)));
template <bool STREAM> __device__ __forceinline__ void store_wide(float *p, const float4 &v) {
  if constexpr (STREAM) {
    const native_f4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<native_f4 *>(p));
  } else {
    *reinterpret_cast<float4 *>(p) = v;
  }
}
template <bool STREAM> __device__ __forceinline__ void store_wide(__half *p, const uint4 &v) {
  if constexpr (STREAM) {
    const native_u4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<native_u4 *>(p));
  } else {
    *reinterpret_cast<uint4 *>(p) = v;
  }
}
template <bool STREAM> __device__ __forceinline__ void store_wide(__half *p, const uint2 &v) {
  if constexpr (STREAM) {
    const native_u2 t = {v.x, v.y};
    __builtin_nontemporal_store(t, reinterpret_cast<native_u2 *>(p));
  } else {
    *reinterpret_cast<uint2 *>(p) = v;
  }
}

template <typename T, int VEC, bool STREAM = true>
__device__ __forceinline__ void store_vec(T *__restrict__ p, const float (&in)[VEC]) {
  if constexpr (VEC == 1) {
    p[0] = from_f32<T>(in[0]);
  } else if constexpr (sizeof(T) == 4) {
    store_wide<STREAM>(p, make_float4(in[0], in[1], in[2], in[3]));
  } else if constexpr (VEC == 4) {
    uint2 raw;
    __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      h[i] = __floats2half2_rn(in[2 * i], in[2 * i + 1]);
    store_wide<STREAM>(p, raw);
  } else {
    uint4 raw;
    __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      h[i] = __floats2half2_rn(in[2 * i], in[2 * i + 1]);
    store_wide<STREAM>(p, raw);
  }
}

// Register-resident copy of VEC elements in their storage format (a half
// vector stays packed: 4 registers for 8 values) with widening on use.
template <typename T, int VEC> struct RawVec;
template <> struct RawVec<float, 4> { float4 v; };
template <> struct RawVec<float, 1> { float v; };
template <> struct RawVec<__half, 8> { uint4 v; };
template <> struct RawVec<__half, 4> { uint2 v; }; // 8-byte access (planes of 4k elements)
template <> struct RawVec<__half, 1> { __half v; };

template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> load_raw(const T *__restrict__ p) {
  RawVec<T, VEC> r;
  if constexpr (VEC == 1) {
    r.v = p[0];
  } else if constexpr (sizeof(T) == 4) {
    r.v = *reinterpret_cast<const float4 *>(p);
  } else if constexpr (VEC == 4) {
    r.v = *reinterpret_cast<const uint2 *>(p);
  } else {
    r.v = *reinterpret_cast<const uint4 *>(p);
  }
  return r;
}

template <typename T, int VEC> __device__ __forceinline__ RawVec<T, VEC> zero_raw() {
  RawVec<T, VEC> r;
  if constexpr (VEC == 1) {
    r.v = from_f32<T>(0.f);
  } else if constexpr (sizeof(T) == 4) {
    r.v = make_float4(0.f, 0.f, 0.f, 0.f);
  } else if constexpr (VEC == 4) {
    r.v = make_uint2(0u, 0u);
  } else {
    r.v = make_uint4(0u, 0u, 0u, 0u);
  }
  return r;
}

template <typename T, int VEC>
__device__ __forceinline__ void unpack(const RawVec<T, VEC> &r, float (&out)[VEC]) {
  if constexpr (VEC == 1) {
    out[0] = to_f32<T>(r.v);
  } else if constexpr (sizeof(T) == 4) {
    out[0] = r.v.x; out[1] = r.v.y; out[2] = r.v.z; out[3] = r.v.w;
  } else {
    const __half2 *h = reinterpret_cast<const __half2 *>(&r.v);
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) {
      const float2 f = __half22float2(h[i]);
      out[2 * i] = f.x;
      out[2 * i + 1] = f.y;
    }
  }
}

// Hides the value of a packed half vector from the optimiser so that the
// widened floats of one phase are not kept alive for the next one (the point
// of keeping the row packed).  No instruction is emitted.
template <typename T, int VEC> __device__ __forceinline__ void keep_packed(RawVec<T, VEC> &r) {
  if constexpr (sizeof(T) == 2 && VEC == 8) {
    asm volatile("" : "+v"(r.v.x), "+v"(r.v.y), "+v"(r.v.z), "+v"(r.v.w));
  } else if constexpr (sizeof(T) == 2 && VEC == 4) {
    asm volatile("" : "+v"(r.v.x), "+v"(r.v.y));
  }
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences
// global memory, i.e. waits for every outstanding global load and store of the
// wave (s_waitcnt vmcnt(0)) before the barrier: loads prefetched for the next
// row and stores of the previous one would all have to land first.  No kernel
// here communicates between threads through global memory, so the barriers
// only need the LDS writes of each wave to have landed (s_waitcnt lgkmcnt(0)).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---------------------------------------------------------------------------
// Element access on packed vectors with the widening folded into the
// arithmetic.  For half data, fma(float(h), a, b) with a half operand taken
// straight from the packed register compiles to ONE v_fma_mix_f32, provided
// the multiplier is not a literal 1.0 (the optimiser would turn the fma into
// an add and need a separate conversion): callers that only want float(h)+b
// pass a 1.0f that arrives as a kernel argument.  raw_sum adds two halves per
// v_dot2_f32_f16.
// ---------------------------------------------------------------------------
typedef _Float16 half2_native __attribute__((ext_vector_type(2)));

// float(x[j]) * a + b for element j of the vector (j is a compile-time
// constant after unrolling).
template <typename T, int VEC>
__device__ __forceinline__ float elem_fma(const RawVec<T, VEC> &r, int j, float a, float b) {
  if constexpr (VEC == 1) {
    return fmaf(to_f32<T>(r.v), a, b);
  } else if constexpr (sizeof(T) == 4) {
    const float x = j == 0 ? r.v.x : j == 1 ? r.v.y : j == 2 ? r.v.z : r.v.w;
    return fmaf(x, a, b);
  } else if constexpr (VEC == 4) {
    const uint32_t w = j < 2 ? r.v.x : r.v.y;
    const half2_native h = __builtin_bit_cast(half2_native, w);
    return fmaf(static_cast<float>((j & 1) ? h.y : h.x), a, b);
  } else {
    const uint32_t w = j < 2 ? r.v.x : j < 4 ? r.v.y : j < 6 ? r.v.z : r.v.w;
    const half2_native h = __builtin_bit_cast(half2_native, w);
    return fmaf(static_cast<float>((j & 1) ? h.y : h.x), a, b);
  }
}

// (x[j] - mean) * istd.  Half data takes the folded one-instruction form
// x*istd + (-mean*istd): its extra error, eps32*|mean|*istd, is far below half
// resolution.  Float data keeps the centred two-instruction form, exact for
// x == mean and insensitive to |mean| >> std.
template <typename T, int VEC>
__device__ __forceinline__ float norm_elem(const RawVec<T, VEC> &r, int j, float mean,
                                           float istd, float nmi) {
  if constexpr (sizeof(T) == 2) {
    return elem_fma<T, VEC>(r, j, istd, nmi);
  } else {
    return (elem_fma<T, VEC>(r, j, 1.0f, 0.f) - mean) * istd;
  }
}

// r when ok, zeros otherwise (branch-free: the load itself is unconditional).
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> raw_or_zero(bool ok, RawVec<T, VEC> r) {
  if constexpr (VEC == 1) {
    r.v = ok ? r.v : from_f32<T>(0.f);
  } else if constexpr (sizeof(T) == 4) {
    r.v.x = ok ? r.v.x : 0.f; r.v.y = ok ? r.v.y : 0.f;
    r.v.z = ok ? r.v.z : 0.f; r.v.w = ok ? r.v.w : 0.f;
  } else if constexpr (VEC == 4) {
    r.v.x = ok ? r.v.x : 0u; r.v.y = ok ? r.v.y : 0u;
  } else {
    r.v.x = ok ? r.v.x : 0u; r.v.y = ok ? r.v.y : 0u;
    r.v.z = ok ? r.v.z : 0u; r.v.w = ok ? r.v.w : 0u;
  }
  return r;
}

// 0xFFFF in each 16-bit half of the result whose half-precision value in w is
// greater than zero (positive, not NaN), 0 elsewhere.  Per half: magnitude
// != 0 (adding 0x7FFF carries into bit 15), magnitude <= 0x7C00 (0xFC00 minus
// it keeps bit 15) and sign clear; neither step crosses the 16-bit boundary.
__device__ __forceinline__ uint32_t half2_gt_zero_mask(uint32_t w) {
  const uint32_t mag = w & 0x7FFF7FFFu;
  const uint32_t bit = (mag + 0x7FFF7FFFu) & (0xFC00FC00u - mag) & ~w & 0x80008000u;
  return (bit >> 15) * 0xFFFFu;
}

// ReLU backward on the storage format: dy where y > 0, zero elsewhere
// (kernel_relu_backward, include/nbla/cuda/utils/relu.cuh:56-62).
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> raw_relu_mask(RawVec<T, VEC> dy, const RawVec<T, VEC> &y) {
  if constexpr (VEC == 1) {
    dy.v = to_f32<T>(y.v) > 0.f ? dy.v : from_f32<T>(0.f);
  } else if constexpr (sizeof(T) == 4) {
    dy.v.x = y.v.x > 0.f ? dy.v.x : 0.f; dy.v.y = y.v.y > 0.f ? dy.v.y : 0.f;
    dy.v.z = y.v.z > 0.f ? dy.v.z : 0.f; dy.v.w = y.v.w > 0.f ? dy.v.w : 0.f;
  } else if constexpr (VEC == 4) {
    dy.v.x &= half2_gt_zero_mask(y.v.x); dy.v.y &= half2_gt_zero_mask(y.v.y);
  } else {
    dy.v.x &= half2_gt_zero_mask(y.v.x); dy.v.y &= half2_gt_zero_mask(y.v.y);
    dy.v.z &= half2_gt_zero_mask(y.v.z); dy.v.w &= half2_gt_zero_mask(y.v.w);
  }
  return dy;
}

// Zeroes the elements of a raw vector outside [lo, hi).
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> raw_keep_range(RawVec<T, VEC> r, int lo, int hi) {
  if constexpr (VEC == 1) {
    if (!(0 >= lo && 0 < hi)) r = zero_raw<T, VEC>();
  } else if constexpr (sizeof(T) == 4) {
    r.v.x = (0 >= lo && 0 < hi) ? r.v.x : 0.f;
    r.v.y = (1 >= lo && 1 < hi) ? r.v.y : 0.f;
    r.v.z = (2 >= lo && 2 < hi) ? r.v.z : 0.f;
    r.v.w = (3 >= lo && 3 < hi) ? r.v.w : 0.f;
  } else {
    uint32_t *w = reinterpret_cast<uint32_t *>(&r.v);
#pragma unroll
    for (int k = 0; k < VEC / 2; ++k) {
      const uint32_t m = ((2 * k >= lo && 2 * k < hi) ? 0x0000ffffu : 0u) |
                         ((2 * k + 1 >= lo && 2 * k + 1 < hi) ? 0xffff0000u : 0u);
      w[k] &= m;
    }
  }
  return r;
}

template <typename T, int VEC, bool STREAM = true>
__device__ __forceinline__ void store_raw(T *__restrict__ p, const RawVec<T, VEC> &r) {
  if constexpr (VEC == 1) {
    p[0] = r.v;
  } else if constexpr (sizeof(T) == 4) {
    store_wide<STREAM>(p, r.v);
  } else if constexpr (VEC == 4) {
    store_wide<STREAM>(p, r.v);
  } else {
    store_wide<STREAM>(p, r.v);
  }
}

// acc + sum of the VEC elements (fp32 accumulation).
template <typename T, int VEC>
__device__ __forceinline__ float raw_sum(const RawVec<T, VEC> &r, float acc) {
  if constexpr (VEC == 1) {
    return acc + to_f32<T>(r.v);
  } else if constexpr (sizeof(T) == 4) {
    return acc + ((r.v.x + r.v.y) + (r.v.z + r.v.w));
  } else {
    const half2_native ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_native, r.v.x), ones, acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_native, r.v.y), ones, acc, false);
    if constexpr (VEC == 8) {
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_native, r.v.z), ones, acc, false);
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_native, r.v.w), ones, acc, false);
    }
    return acc;
  }
}

// VEC consecutive float parameters (gamma/beta style), p aligned to 16 bytes
// when VEC > 1.
template <int VEC>
__device__ __forceinline__ void load_param_vec(const float *__restrict__ p,
                                               float (&out)[VEC]) {
  if constexpr (VEC == 1) {
    out[0] = p[0];
  } else {
#pragma unroll
    for (int i = 0; i < VEC / 4; ++i) {
      const float4 v = reinterpret_cast<const float4 *>(p)[i];
      out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
    }
  }
}

// ---------------------------------------------------------------------------
// Division by a runtime constant without the integer divider: q = n / d for
// 0 <= n < 2^31 and 1 <= d < 2^31 (round-up multiplier, 64-bit product).
// ---------------------------------------------------------------------------
struct FastDiv {
  uint32_t d;
  uint32_t mul;
  uint32_t shift;
  __host__ FastDiv() : d(1), mul(0), shift(0) {}
  __host__ explicit FastDiv(uint32_t divisor) : d(divisor) {
    if (divisor <= 1) {
      d = 1; mul = 0; shift = 0;
      return;
    }
    uint32_t s = 0;
    while ((1ull << s) < divisor) ++s;           // s = ceil(log2 d)
    const uint64_t m = ((1ull << (31 + s)) + divisor - 1) / divisor; // < 2^32
    mul = static_cast<uint32_t>(m);
    shift = s;
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
    if (d == 1) return n;
    return static_cast<uint32_t>((static_cast<uint64_t>(n) * mul) >> 31) >> shift;
  }
};

// ---------------------------------------------------------------------------
// Wavefront-64 all-reduce (sum).  Steps 1,2,4,8 stay inside a 16-lane DPP row:
// quad_perm xor1, quad_perm xor2, row_half_mirror, row_mirror.  After them each
// row is uniform and the four row values are fetched with lane reads, so the
// result is wave-uniform and identical in every lane.
// ---------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf,
                                         0xf, true));
}

__device__ __forceinline__ float read_lane(float v, int lane) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);  // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v); // row_half_mirror
  v += dpp_move<0x140>(v); // row_mirror
  return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

// v + (v of lane ^ OFF), OFF a power of two below 64, without the LDS crossbar
// where the vector unit has a path of its own: quad_perm for 1 and 2, a row
// rotation for 8 (lane (i + 8) % 16 of the 16-lane row is lane i ^ 8), and
// gfx950's row and half-wave swaps for 16 and 32 (with both operands the same
// register, v_permlane16_swap leaves rows (r0, r0, r2, r2) and (r1, r1, r3, r3),
// v_permlane32_swap halves (lo, lo) and (hi, hi): their sum is the butterfly
// step, in every lane the same two addends).  ds_bpermute for 4.  Sixteen waves
// folding 8 values over 3 steps through ds_bpermute kept a CU's LDS busy for
// 1.4 us; on these paths the same fold is 60 vector instructions per wave.
// (Written as inline assembly: the builtins of ROCm 7.2's compiler,
// __builtin_amdgcn_permlane16_swap / 32_swap, return the first register for
// both halves of their result pair.  The swap works in place on two registers;
// the idle cycles around it keep it clear of the vector results before it and
// of its readers, which the compiler's hazard pass cannot see inside asm.)
__device__ __forceinline__ float swap_add16(float v) {
  float a = v, b = v;
  asm volatile("s_nop 3\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
__device__ __forceinline__ float swap_add32(float v) {
  float a = v, b = v;
  asm volatile("s_nop 3\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
template <int OFF> __device__ __forceinline__ float xor_add(float v) {
  static_assert(OFF == 1 || OFF == 2 || OFF == 4 || OFF == 8 || OFF == 16 || OFF == 32, "lane bit");
  if constexpr (OFF == 1) {
    return v + dpp_move<0xB1>(v);
  } else if constexpr (OFF == 2) {
    return v + dpp_move<0x4E>(v);
  } else if constexpr (OFF == 8) {
    return v + dpp_move<0x128>(v); // row_ror:8
  } else if constexpr (OFF == 16) {
    return swap_add16(v);
  } else if constexpr (OFF == 32) {
    return swap_add32(v);
  } else {
    return v + __shfl_xor(v, OFF);
  }
}

// Butterfly sums of N values at once over the lane bits lo, 2 lo, ... 32
// (lanes_sum_from: every lane ends with the sum over the lanes that differ
// from it in those bits only) or 1, 2, ... hi / 2 (lanes_sum_below); lo and hi
// are powers of two known at run time, uniform over the wave.  A step at a time
// for all values, so that the cross-lane operations of a step overlap.
template <int N> __device__ __forceinline__ void lanes_sum_from(float (&v)[N], uint32_t lo) {
#define NBLAHIP_STEP(OFF)                                  \
  if (lo <= (OFF)) {                                       \
    _Pragma("unroll") for (int j = 0; j < N; ++j) v[j] = xor_add<OFF>(v[j]); \
  }
  NBLAHIP_STEP(1)
  NBLAHIP_STEP(2)
  NBLAHIP_STEP(4)
  NBLAHIP_STEP(8)
  NBLAHIP_STEP(16)
  NBLAHIP_STEP(32)
#undef NBLAHIP_STEP
}
template <int N> __device__ __forceinline__ void lanes_sum_below(float (&v)[N], uint32_t hi) {
#define NBLAHIP_STEP(OFF)                                  \
  if (hi > (OFF)) {                                        \
    _Pragma("unroll") for (int j = 0; j < N; ++j) v[j] = xor_add<OFF>(v[j]); \
  }
  NBLAHIP_STEP(1)
  NBLAHIP_STEP(2)
  NBLAHIP_STEP(4)
  NBLAHIP_STEP(8)
  NBLAHIP_STEP(16)
  NBLAHIP_STEP(32)
#undef NBLAHIP_STEP
}
__device__ __forceinline__ float lanes_sum_from(float x, uint32_t lo) {
  float v[1] = {x};
  lanes_sum_from<1>(v, lo);
  return v[0];
}
__device__ __forceinline__ float lanes_sum_below(float x, uint32_t hi) {
  float v[1] = {x};
  lanes_sum_below<1>(v, hi);
  return v[0];
}

// Sum over aligned groups of G = 4, 8, 16 or 32 adjacent lanes (every lane of
// a group returns the group's sum): the first steps of wave_sum, and one lane
// exchange between the two 16-lane rows for G = 32.  Lanes of a group must be
// active together.
template <int G> __device__ __forceinline__ float group_sum(float v) {
  static_assert(G == 4 || G == 8 || G == 16 || G == 32, "sub-wave group size");
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  if constexpr (G >= 8) v += dpp_move<0x141>(v);
  if constexpr (G >= 16) v += dpp_move<0x140>(v);
  if constexpr (G == 32) v = xor_add<16>(v);
  return v;
}

// Sum over a group of TPR threads that share a row.  TPR < 64: several rows
// per wave.  TPR == 64: one wave.  TPR > 64: the block is exactly one row
// (blockDim.x == TPR); `lds` holds TPR/64 floats and is reused, so the call
// ends with a barrier-protected read.
template <int TPR>
__device__ __forceinline__ float row_sum(float v, float *lds) {
  if constexpr (TPR < kWave) {
    return group_sum<TPR>(v);
  } else if constexpr (TPR == kWave) {
    return wave_sum(v);
  } else {
    v = wave_sum(v);
    constexpr int NW = TPR / kWave;
    const int wave = threadIdx.x / kWave;
    lds_barrier(); // previous readers of lds are done
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
    lds_barrier();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) total += lds[i];
    return total;
  }
}

// Two sums at once (halves the number of barriers).
template <int TPR>
__device__ __forceinline__ void row_sum2(float &a, float &b, float *lds) {
  if constexpr (TPR < kWave) {
    a = group_sum<TPR>(a);
    b = group_sum<TPR>(b);
    return;
  } else {
    a = wave_sum(a);
    b = wave_sum(b);
  }
  if constexpr (TPR > kWave) {
    constexpr int NW = TPR / kWave;
    const int wave = threadIdx.x / kWave;
    lds_barrier();
    if ((threadIdx.x & (kWave - 1)) == 0) {
      lds[2 * wave] = a;
      lds[2 * wave + 1] = b;
    }
    lds_barrier();
    float ta = 0.f, tb = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      ta += lds[2 * i];
      tb += lds[2 * i + 1];
    }
    a = ta;
    b = tb;
  }
}

// ---------------------------------------------------------------------------
// Welford state and the Chan/Golub/LeVeque merge (the reference's
// include/nbla/cuda/utils/reduce_ops/welford.cuh:80-97).  n is kept in float:
// exact up to 2^24 per partial, which every launch configuration respects.
// ---------------------------------------------------------------------------
struct Welford {
  float mean, m2, n;
};

// 1/x to within one ulp (v_rcp_f32); the merge weights do not need the
// correctly rounded quotient and the full division costs ten instructions.
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ Welford welford_merge(const Welford &a, const Welford &b) {
  const float n = a.n + b.n;
  if (n == 0.f) return Welford{0.f, 0.f, 0.f};
  const float inv = fast_rcp(n);
  const float d = b.mean - a.mean;
  Welford r;
  r.mean = a.mean + d * (b.n * inv);
  r.m2 = a.m2 + b.m2 + d * d * (a.n * b.n * inv);
  r.n = n;
  return r;
}

// Merge a chunk of CNT values v[] (CNT >= 1, compile-time bound, `cnt` valid)
// into acc: chunk mean and centred M2 are formed in registers first, so only
// one reciprocal is spent per chunk.
template <int CNT>
__device__ __forceinline__ void welford_add_chunk(Welford &acc, const float (&v)[CNT],
                                                  int cnt) {
  if (cnt <= 0) return;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CNT; ++i) s += (i < cnt) ? v[i] : 0.f;
  const float fc = static_cast<float>(cnt);
  const float cm = s * fast_rcp(fc);
  float m2 = 0.f;
#pragma unroll
  for (int i = 0; i < CNT; ++i) {
    const float d = v[i] - cm;
    m2 += (i < cnt) ? d * d : 0.f;
  }
  acc = welford_merge(acc, Welford{cm, m2, fc});
}

// The same with an arbitrary subset of the chunk valid (ok[i]).
template <int CNT>
__device__ __forceinline__ void welford_add_chunk_masked(Welford &acc, const float (&v)[CNT],
                                                         const bool (&ok)[CNT]) {
  float s = 0.f;
  int cnt = 0;
#pragma unroll
  for (int i = 0; i < CNT; ++i) {
    s += ok[i] ? v[i] : 0.f;
    cnt += ok[i] ? 1 : 0;
  }
  if (cnt == 0) return;
  const float fc = static_cast<float>(cnt);
  const float cm = s * fast_rcp(fc);
  float m2 = 0.f;
#pragma unroll
  for (int i = 0; i < CNT; ++i) {
    const float d = v[i] - cm;
    m2 += ok[i] ? d * d : 0.f;
  }
  acc = welford_merge(acc, Welford{cm, m2, fc});
}

__device__ __forceinline__ Welford wave_welford(Welford w) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    Welford o;
    o.mean = __shfl_xor(w.mean, off);
    o.m2 = __shfl_xor(w.m2, off);
    o.n = __shfl_xor(w.n, off);
    // Keep the operand order identical in both partners so they agree bitwise.
    const bool low = (threadIdx.x & off) == 0;
    w = low ? welford_merge(w, o) : welford_merge(o, w);
  }
  return w;
}

// Block-wide Welford merge; lds holds 3*(blockDim.x/64) floats.  Every thread
// returns the same merged state.
__device__ __forceinline__ Welford block_welford(Welford w, float *lds) {
  w = wave_welford(w);
  const int nw = blockDim.x / kWave;
  if (nw == 1) return w;
  const int wave = threadIdx.x / kWave;
  lds_barrier();
  if ((threadIdx.x & (kWave - 1)) == 0) {
    lds[3 * wave] = w.mean;
    lds[3 * wave + 1] = w.m2;
    lds[3 * wave + 2] = w.n;
  }
  lds_barrier();
  Welford t{lds[0], lds[1], lds[2]};
  for (int i = 1; i < nw; ++i)
    t = welford_merge(t, Welford{lds[3 * i], lds[3 * i + 1], lds[3 * i + 2]});
  return t;
}

// Block-wide sum of two values; lds holds 2*(blockDim.x/64) floats.
__device__ __forceinline__ void block_sum2(float &a, float &b, float *lds) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int nw = blockDim.x / kWave;
  if (nw == 1) return;
  const int wave = threadIdx.x / kWave;
  lds_barrier();
  if ((threadIdx.x & (kWave - 1)) == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  lds_barrier();
  float ta = 0.f, tb = 0.f;
  for (int i = 0; i < nw; ++i) {
    ta += lds[2 * i];
    tb += lds[2 * i + 1];
  }
  a = ta;
  b = tb;
}

__device__ __forceinline__ float inv_std(float var, float eps) {
  return 1.0f / sqrtf(var + eps);
}

// Calls f(i, lds[i * stride], lds[i * stride + 1]) for i = 0 .. n - 1 in order,
// with the LDS reads of eight steps in flight together: a loop that reads as it
// goes pays an LDS round trip per step (2 us for 16 partners' partial sums).
template <typename F>
__device__ __forceinline__ void for_pairs_in_order(const float *lds, int stride, int n, F f) {
  for (int i0 = 0; i0 < n; i0 += 8) {
    float v0[8], v1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = min(i0 + i, n - 1);
      v0[i] = lds[idx * stride];
      v1[i] = lds[idx * stride + 1];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i0 + i < n) f(i0 + i, v0[i], v1[i]);
    }
  }
}

} // namespace nblahip
