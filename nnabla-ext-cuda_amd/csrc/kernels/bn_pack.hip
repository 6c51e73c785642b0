// BatchNormalization training for planes that are not a whole number of
// 16-byte vectors (7x7 and, in half, 14x14: the late stages of a ResNet), with
// a PACK of neighbouring channels held on one CU.
//
// x is [N][C][HW].  A plane of 49 half elements is 98 bytes: a channel's planes
// start at odd addresses, so a block that owns one channel reads them element
// by element, or in vectors that it shares with the neighbouring channels and
// masks.  But G = 16 / gcd(HW * sizeof(T), 16) neighbouring channels (2, 4 or 8)
// form a segment of G * HW elements that IS a whole number of vectors and
// starts on a 16-byte boundary in every sample (C a multiple of G).  A
// 1024-thread block takes such a pack: thread t owns vector t % nvs of the
// segment in the samples t / nvs + k * rpi (nvs vectors per segment, rpi =
// 1024 / nvs samples per sweep), NR vectors in registers and NS more in LDS as
// in bn_onchip.hip.  Element j of a thread's vectors is always the same
// position of the same channel, so the thread keeps one accumulator per
// element; the block adds them per channel through LDS in a fixed order
// (samples, then the positions of a plane).  x crosses the memory system once:
// 2 S forward; the backward holds x and as much of dy as LDS takes beside the
// reduction's scratch and reads the rest of dy a second time (3 S to 3.5 S).
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"

namespace nblahip {

namespace {

constexpr int kPackMaxG = 8;     // channels of a pack
constexpr int kPackMaxNvs = 128; // vectors of a segment (at least 8 samples per sweep)

struct BnPackArgs {
  const void *x;
  void *y;
  const float *gamma, *beta;
  float *mean, *var, *rmean, *rvar;
  uint32_t C, hw, G;
  uint32_t N;          // samples
  FastDiv nvs;         // vectors per segment = G * hw / VEC
  FastDiv hwd;         // hw, for element -> channel of the pack
  uint32_t rpi;        // samples per sweep = 1024 / nvs
  uint32_t per_xcd;    // packs per XCD when neighbouring packs share an XCD, else 0
  uint32_t edge_lines; // samples lie a whole number of 128-byte lines apart
  uint32_t active;     // threads that own a vector = rpi * nvs
  uint32_t row_stride; // elements between samples = C * hw
  float inv_N, unbias, decay, eps, one;
  // backward
  const void *dy;
  void *dx;                  // may be null
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;     // may be null
  int accum_dx, accum_g, accum_b;
};

// Pack of block b.  Workgroups go to the 8 XCDs round-robin by index; the
// segments of neighbouring packs meet in the 128-byte lines at their ends, so
// neighbouring packs run on the same XCD (one L2 fetches such a line once, and
// merges the two partial writes to it).
__device__ __forceinline__ uint32_t pack_of_block(const BnPackArgs &a, uint32_t b) {
  return a.per_xcd ? (b % 8u) * a.per_xcd + b / 8u : b;
}

// Whether the thread's vector lies in a 128-byte line that its segment shares
// with a neighbouring pack's (the same in every sample when the samples lie
// whole lines apart).  Such vectors are written with ordinary stores, which
// the XCD's L2 merges with the neighbour's part of the line; non-temporal
// stores of line pieces go to memory piece by piece (a 51 MB copy in this
// block shape: 22.5 -> 21.5 us).
template <typename T, int VEC>
__device__ __forceinline__ bool pack_edge_vector(const BnPackArgs &a, const T *p, uint32_t v) {
  if (!a.edge_lines) return false;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  const uintptr_t first = addr - static_cast<uintptr_t>(v) * 16u, end = first + a.nvs.d * 16u;
  const uintptr_t line = addr >> 7;
  return line < ((first + 127u) >> 7) || line >= (end >> 7);
}

// Per-channel totals of the threads' per-element values: tot[g] = sum of v[j]
// over every thread and element that lies in channel g of the pack.  cols
// holds the values as [sample of the sweep][position in the segment] (thread
// t's vector is at t * VEC); a thread per position adds the samples in order,
// a wave per channel adds the positions of its plane.  The order is fixed:
// the same bits in every run.  Ends with a barrier (tot is readable).
template <int VEC>
__device__ __forceinline__ void pack_channel_sums(const float (&v)[VEC], const BnPackArgs &a,
                                                  bool owner, float *cols, float *csum,
                                                  float *tot) {
  const uint32_t t = threadIdx.x;
  lds_barrier(); // earlier readers of cols / csum / tot are done
  if (owner) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) cols[t * VEC + j] = v[j];
  } else if (t < a.active) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) cols[t * VEC + j] = 0.f;
  }
  lds_barrier();
  const uint32_t seg = a.nvs.d * VEC;
  for (uint32_t j = t; j < seg; j += kOnchipBlock) {
    // (four sums side by side: one wait for four reads instead of one each)
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint32_t r = 0;
    for (; r + 4 <= a.rpi; r += 4) {
      s0 += cols[r * seg + j];
      s1 += cols[(r + 1) * seg + j];
      s2 += cols[(r + 2) * seg + j];
      s3 += cols[(r + 3) * seg + j];
    }
    for (; r < a.rpi; ++r) s0 += cols[r * seg + j];
    csum[j] = (s0 + s1) + (s2 + s3);
  }
  lds_barrier();
  const uint32_t wave = t / kWave, lane = t % kWave;
  for (uint32_t g = wave; g < a.G; g += kOnchipBlock / kWave) {
    float s = 0.f;
    for (uint32_t i = lane; i < a.hw; i += kWave) s += csum[g * a.hw + i];
    s = wave_sum(s);
    if (lane == 0) tot[g] = s;
  }
  lds_barrier();
}

} // namespace

template <typename T, int VEC, int NR, int NS>
__global__ void __launch_bounds__(kOnchipBlock)
bn_pack_fwd_kernel(const BnPackArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float cols[kOnchipBlock * VEC];
  __shared__ float csum[kPackMaxNvs * VEC];
  __shared__ float tot[kPackMaxG];
  __shared__ float fin[3 * kPackMaxG]; // mean, scale, shift (float data: beta) per channel
  const uint32_t t = threadIdx.x;
  const uint32_t c0 = pack_of_block(a, blockIdx.x) * a.G;
  // gamma and beta of channel t of the pack, asked for ahead of the tensor
  // (and the running statistics it updates: behind the block sums each load
  // would cost a memory round trip of its own)
  float gamma_t = 1.f, beta_t = 0.f, rmean_t = 0.f, rvar_t = 0.f;
  if (t < a.G) {
    if (a.gamma) gamma_t = a.gamma[c0 + t];
    if (a.beta) beta_t = a.beta[c0 + t];
    if (a.rmean) rmean_t = a.rmean[c0 + t];
    if (a.rvar) rvar_t = a.rvar[c0 + t];
  }
  // thread -> (sample of the sweep, vector of the segment); a thread without a
  // vector of its own reads thread 0's and stays out of sums and stores
  uint32_t r = a.nvs.div(t);
  const bool owner = t < a.active && r < a.N;
  const uint32_t tt = owner ? t : 0u;
  r = owner ? r : 0u;
  const uint32_t v = tt - r * a.nvs.d;
  const int rv = owner ? static_cast<int>(r) : 0x3fffffff;
  const size_t base = static_cast<size_t>(r) * a.row_stride + static_cast<size_t>(c0) * a.hw + v * VEC;
  const size_t step = static_cast<size_t>(a.rpi) * a.row_stride;
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  T *__restrict__ y = static_cast<T *>(a.y) + base;
  // (slot k holds a vector: the thread's sample against a scalar, no register per slot)
  auto holds = [&](int k) { return rv < static_cast<int>(a.N) - k * static_cast<int>(a.rpi); };

  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) parked[k] = load_raw<T, VEC>(holds(NR + k) ? x + (NR + k) * step : x);
#pragma unroll
    for (int k = 0; k < NR; ++k) raw[k] = load_raw<T, VEC>(holds(k) ? x + k * step : x);
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };

  // ---- statistics: per thread and element a running (mean, m2) over the
  // thread's samples (Welford, the reciprocal counts are constants of the
  // unrolled code), each slot as its load arrives: ahead of the block's first
  // barrier a wave's arithmetic hides behind the other waves' loads, and only
  // the last slot's is left when the last load lands (sums about the thread's
  // own mean, a second pass over the registers once all loads are in, cost
  // 2.3 us of [256,2048,7,7] half's 28.5).  Per channel then
  // mean = sum n*mean_t / count and m2 = sum (m2_t + n*(mean_t - mean)^2).
  float m[VEC], q[VEC];
  {
    float mu_t[VEC], m2[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) mu_t[j] = m2[j] = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (holds(k)) {
        const RawVec<T, VEC> x_k = slot(k);
        const float rk = 1.0f / static_cast<float>(k + 1);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(x_k, j, a.one, -mu_t[j]);
          mu_t[j] = fmaf(d, rk, mu_t[j]);
          m2[j] = fmaf(d, elem_fma<T, VEC>(x_k, j, a.one, -mu_t[j]), m2[j]);
        }
      }
    }
    const float nt = owner ? static_cast<float>((a.N - 1u - r) / a.rpi + 1u) : 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) m[j] = nt * mu_t[j];
    pack_channel_sums<VEC>(m, a, owner, cols, csum, tot);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float e = mu_t[j] - tot[a.hwd.div(v * VEC + j)] * a.inv_N;
      q[j] = fmaf(nt * e, e, m2[j]);
    }
  }
  const float mean_t = t < a.G ? tot[t] * a.inv_N : 0.f;
  pack_channel_sums<VEC>(q, a, owner, cols, csum, tot);
  if (t < a.G) {
    const float var_t = tot[t] * a.inv_N;
    a.mean[c0 + t] = mean_t;
    a.var[c0 + t] = var_t;
    if (a.rmean) a.rmean[c0 + t] = a.decay * rmean_t + (1.f - a.decay) * mean_t;
    if (a.rvar) a.rvar[c0 + t] = a.decay * rvar_t + (1.f - a.decay) * var_t * a.unbias;
    const float sc = gamma_t * inv_std(var_t, a.eps);
    fin[t] = mean_t;
    fin[kPackMaxG + t] = sc;
    fin[2 * kPackMaxG + t] = sizeof(T) == 2 ? fmaf(-mean_t, sc, beta_t) : beta_t;
  }
  lds_barrier();

  // ---- normalize what the block holds
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  const bool edge = pack_edge_vector<T, VEC>(a, y, v);
  float mu[VEC], sc[VEC], sh[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t g = a.hwd.div(v * VEC + j);
    mu[j] = fin[g];
    sc[j] = fin[kPackMaxG + g];
    sh[j] = fin[2 * kPackMaxG + g];
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (holds(k)) {
      const RawVec<T, VEC> x_k = slot(k);
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(x_k, j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(x_k, j, a.one, -mu[j]), sc[j], sh[j]);
        }
      }
      if (edge) {
        store_vec<T, VEC, false>(y + k * step, o);
      } else {
        store_vec<T, VEC>(y + k * step, o);
      }
    }
  }
}

// Backward (batch statistics).  With xh = (x-mean)*istd per channel:
//   sdx = sum dy*xh (= dgamma), sdy = sum dy (= dbeta),
//   dx = dy*g*istd + xh*cA + cb,  cA = -istd*g*sdx/N + 2*dvar*std/N,
//   cb = -g*sdy*istd/N + dmean/N.
// x stays in registers (NL vectors per thread); dy is read in batches of B
// vectors, its first ND vectors per thread wait in LDS for the second pass, the
// others are read again.
template <typename T, int VEC, int NL, int ND, int B>
__global__ void __launch_bounds__(kOnchipBlock)
bn_pack_bwd_kernel(const BnPackArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  __shared__ uint4 park[ND > 0 ? ND * kOnchipBlock : 1];
  __shared__ float cols[kOnchipBlock * VEC];
  __shared__ float csum[kPackMaxNvs * VEC];
  __shared__ float tot[kPackMaxG];
  __shared__ float par[2 * kPackMaxG];  // mean, var per channel of the pack
  __shared__ float coef[4 * kPackMaxG]; // mean, g*istd, A2, B2
  const uint32_t t = threadIdx.x;
  const uint32_t c0 = pack_of_block(a, blockIdx.x) * a.G;
  // The parameters of channel t of the pack, asked for ahead of the tensor.
  float p_mean = 0.f, p_var = 1.f, p_gamma = 1.f, p_dvar = 0.f, p_dmean = 0.f;
  if (t < a.G) {
    p_mean = a.mean[c0 + t];
    p_var = a.var[c0 + t];
    if (a.gamma) p_gamma = a.gamma[c0 + t];
    if (a.dvar) p_dvar = a.dvar[c0 + t];
    if (a.dmean) p_dmean = a.dmean[c0 + t];
  }
  uint32_t r = a.nvs.div(t);
  const bool owner = t < a.active && r < a.N;
  const uint32_t tt = owner ? t : 0u;
  r = owner ? r : 0u;
  const uint32_t v = tt - r * a.nvs.d;
  const int rv = owner ? static_cast<int>(r) : 0x3fffffff;
  // (element offsets fit 32 bits: the C-ABI admits tensors below 2^31 elements)
  const uint32_t base = r * a.row_stride + c0 * a.hw + v * VEC;
  const uint32_t step = a.rpi * a.row_stride;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.dx);
  auto holds = [&](int k) { return rv < static_cast<int>(a.N) - k * static_cast<int>(a.rpi); };

  RawVec<T, VEC> xr[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) xr[k] = load_raw<T, VEC>(x + (holds(k) ? base + k * step : base));
  if (t < a.G) {
    par[t] = p_mean;
    par[kPackMaxG + t] = p_var;
  }
  lds_barrier();
  float mean[VEC], istd[VEC], nmi[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t g = a.hwd.div(v * VEC + j);
    mean[j] = par[g];
    istd[j] = 1.0f / sqrtf(par[kPackMaxG + g] + a.eps);
    nmi[j] = -mean[j] * istd[j];
  }

  // ---- pass 1: per element (sum dy*xh, sum dy), samples ascending
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t b1 = fresh_after(base, sdx[0]);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) d[i] = load_raw<T, VEC>(dy + (holds(k) ? b1 + k * step : b1));
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        if (k < ND) park[(k < ND ? k : 0) * kOnchipBlock + t] = __builtin_bit_cast(uint4, d[i]);
        if (holds(k)) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float xh = norm_elem<T, VEC>(xr[k], j, mean[j], istd[j], nmi[j]);
            sdx[j] = elem_fma<T, VEC>(d[i], j, xh, sdx[j]);
            sdy[j] = elem_fma<T, VEC>(d[i], j, a.one, sdy[j]);
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0); // the next batch's loads stay below: hoisted, the batches add up
  }
  pack_channel_sums<VEC>(sdx, a, owner, cols, csum, tot);
  const float tx = t < a.G ? tot[t] : 0.f;
  pack_channel_sums<VEC>(sdy, a, owner, cols, csum, tot);
  if (t < a.G) {
    const float ty = tot[t];
    if (a.dgamma) a.dgamma[c0 + t] = tx + (a.accum_g ? a.dgamma[c0 + t] : 0.f);
    if (a.dbeta) a.dbeta[c0 + t] = ty + (a.accum_b ? a.dbeta[c0 + t] : 0.f);
    const float vpe = p_var + a.eps;
    const float is = 1.0f / sqrtf(vpe);
    const float cA = -is * p_gamma * tx * a.inv_N + (a.dvar ? 2.f * p_dvar * (vpe * is) * a.inv_N : 0.f);
    const float cb = -p_gamma * ty * is * a.inv_N + (a.dmean ? p_dmean * a.inv_N : 0.f);
    coef[t] = p_mean;
    coef[kPackMaxG + t] = p_gamma * is;
    coef[2 * kPackMaxG + t] = is * cA;
    coef[3 * kPackMaxG + t] = sizeof(T) == 2 ? fmaf(-p_mean * is, cA, cb) : cb;
  }
  if (dx == nullptr) return;
  lds_barrier();

  // ---- pass 2: dx = dy*gi + (x - mean)*A2 + B2  (half: x*A2 + B2, one mixed fma)
#pragma unroll
  for (int k = 0; k < NL; ++k) forget<T, VEC>(xr[k]);
  const bool edge = pack_edge_vector<T, VEC>(a, dx + base, v);
  float gi[VEC], A2[VEC], B2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t g = a.hwd.div(v * VEC + j);
    mean[j] = coef[g];
    gi[j] = coef[kPackMaxG + g];
    A2[j] = coef[2 * kPackMaxG + g];
    B2[j] = coef[3 * kPackMaxG + g];
  }
  auto emit = [&](const RawVec<T, VEC> &xv, const RawVec<T, VEC> &dv, uint32_t off) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float xt;
      if constexpr (sizeof(T) == 2) {
        xt = elem_fma<T, VEC>(xv, j, A2[j], B2[j]);
      } else {
        xt = fmaf(elem_fma<T, VEC>(xv, j, a.one, -mean[j]), A2[j], B2[j]);
      }
      o[j] = elem_fma<T, VEC>(dv, j, gi[j], xt);
    }
    T *dst = dx + off;
    if (a.accum_dx) {
      float old[VEC];
      load_vec<T, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] += old[j];
    }
    if (edge) {
      store_vec<T, VEC, false>(dst, o);
    } else {
      store_vec<T, VEC>(dst, o);
    }
  };
#pragma unroll
  for (int k = 0; k < ND && k < NL; ++k) {
    if (holds(k)) {
      const RawVec<T, VEC> dv = __builtin_bit_cast(RawVec<T, VEC>, park[k * kOnchipBlock + t]);
      emit(xr[k], dv, base + k * step);
    }
  }
  float lastv = B2[0];
#pragma unroll
  for (int k0 = ND; k0 < NL; k0 += B) {
    const uint32_t b2 = fresh_after(base, lastv);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) d[i] = load_raw<T, VEC>(dy + (holds(k) ? b2 + k * step : b2));
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL && holds(k)) {
        emit(xr[k < NL ? k : 0], d[i], b2 + k * step);
        lastv = __builtin_bit_cast(float, __builtin_bit_cast(uint4, d[i]).x);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

namespace {

template <typename T, int VEC>
int run_pack_fwd(int nl, const BnPackArgs &a, unsigned grid, hipStream_t st) {
#define PACK_CASE(NR, NS)                                                                        \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH("bn_pack_fwd_kernel", (bn_pack_fwd_kernel<T, VEC, NR, NS>), dim3(grid),       \
                   dim3(kOnchipBlock), 0, st, a);                                                \
    return last_launch_status();                                                                 \
  }
  PACK_CASE(2, 0)
  PACK_CASE(4, 0)
  PACK_CASE(7, 0)
  PACK_CASE(10, 0)
  PACK_CASE(13, 0)
  PACK_CASE(16, 0)
  PACK_CASE(16, 3)
  PACK_CASE(16, 5)
#undef PACK_CASE
  return NBLAHIP_EINVAL;
}

constexpr int kPackFwdMax = 21; // vectors per thread the forward holds
constexpr int kPackBwdMax = 13; // ... and the backward (x in registers)

template <typename T, int VEC>
int run_pack_bwd(int nl, const BnPackArgs &a, unsigned grid, hipStream_t st) {
  // dy beside the reduction's scratch (32 KB half, 16 KB float) in LDS
  constexpr int kPark = sizeof(T) == 2 ? 7 : 8;
  constexpr int kB = sizeof(T) == 2 ? 2 : 4;
#define PACK_CASE(NL)                                                                            \
  if (nl <= (NL)) {                                                                              \
    NBLAHIP_LAUNCH("bn_pack_bwd_kernel",                                                         \
                   (bn_pack_bwd_kernel<T, VEC, NL, ((NL) < kPark ? (NL) : kPark), kB>),          \
                   dim3(grid), dim3(kOnchipBlock), 0, st, a);                                    \
    return last_launch_status();                                                                 \
  }
  PACK_CASE(2)
  PACK_CASE(4)
  PACK_CASE(7)
  PACK_CASE(10)
  PACK_CASE(13)
#undef PACK_CASE
  return NBLAHIP_EINVAL;
}

// Shape test and the arguments both directions share; nl = vectors per thread.
bool pack_args(const BnProblem &p, bool backward, BnPackArgs &a, int &nl) {
  if (!tune_int("BN_PACK", 1)) return false;
  if (p.size2 <= 1 || p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  const int esz = p.dtype == NBLAHIP_F16 ? 2 : 4;
  const int vec = 16 / esz;
  const int64_t plane_bytes = p.size2 * esz;
  if (plane_bytes % 16 == 0) return false; // whole vectors per plane: the other kernels' case
  int64_t G = 16;
  while (plane_bytes % G != 0) G >>= 1; // gcd(plane_bytes, 16)
  G = 16 / G;                           // 2, 4 or 8 channels to a whole number of vectors
  if (G > kPackMaxG || p.C % G != 0) return false;
  if (!aligned16(p.x) || (p.out && !aligned16(p.out)) || (backward && !aligned16(p.dy))) return false;
  const int64_t nvs = G * plane_bytes / 16;
  if (nvs > kPackMaxNvs) return false;
  const int64_t rpi = kOnchipBlock / nvs;
  nl = static_cast<int>((p.size0 + rpi - 1) / rpi);
  if (nl > (backward ? kPackBwdMax : kPackFwdMax)) return false;
  if (p.size0 * p.C * p.size2 >= (int64_t{1} << 31)) return false;
  // Packs of two channels (half planes of 4k + 2 elements, 14x14) have 8-byte
  // vectors as their alternative, which do as well - but for the backward of
  // channels beyond the row kernels' registers, which reads dy twice there
  // ([256,1024,14,14] half backward 87.8 -> 69.1 us; forward 55.4 / 55.0;
  // [64,1024,14,14] 16.7 / 19.2 -> 19.4 / 20.9 us).
  if (G == 2 && !(backward && p.size0 * (p.size2 / 4) > 8 * kOnchipBlock)) return false;
  // A block is alone on its CU, and still a few packs beat the three launches
  // of the masked split reduction ([96,240,7,7] half, 30 packs: 18.4 vs 27.0 us
  // of kernel time forward + backward).  Channels of up to 4096 elements, which
  // the row kernels take element by element in one launch, want a pack for
  // every CU ([64,512,7,7] half, 64 packs: 7.7 / 7.7 -> 8.5 / 9.2 us;
  // [32,256,7,7]: rows 8.2 us, packs 12.7; [32,1024,7,7], 128 packs: rows 10.8,
  // packs 13.5; [64,2048,7,7], 256 packs: 17.6 / 20.8 -> 10.8 / 11.5 us).
  const bool short_channels = p.size0 * p.size2 <= 4096;
  const int min_pct = short_channels ? tune_int("BN_PACK_SHORT_MIN_PCT", 100) : tune_int("BN_PACK_MIN_PCT", 1);
  if ((p.C / G) * 100 < static_cast<int64_t>(device_cus()) * min_pct) return false;
  // Few packs of long channels, where a block per channel can hold the channel:
  // that many more blocks win (forward / backward us, packs against the masked
  // block per channel or, shorter channels, the row kernels: [256,256,7,7] half,
  // 32 packs, 18.6 / 20.4 vs 15.6 / 13.4; [128,160,7,7] half, 20 packs, 11.1 / 11.7
  // vs 6.6 / 6.4; [256,320,7,7] half, 40 packs, 19.1 / 20.5 vs 17.3 / 18.7;
  // [128,160,7,7] float, 40 packs, 11.0 / 11.1 vs 7.5 / 8.7; from 64 packs on the
  // packs are ahead, [256,512,7,7] half 19.1 / 21.0 vs 19.6 / 23.2).
  if (!short_channels &&
      (p.C / G) * 100 < static_cast<int64_t>(device_cus()) * tune_int("BN_PACK_MIN_PCT_MASKED", 16) &&
      bn_masked_takes(p, backward))
    return false;
  a = BnPackArgs{};
  a.x = p.x;
  a.gamma = p.gamma;
  a.C = static_cast<uint32_t>(p.C);
  a.hw = static_cast<uint32_t>(p.size2);
  a.G = static_cast<uint32_t>(G);
  a.N = static_cast<uint32_t>(p.size0);
  a.nvs = FastDiv(static_cast<uint32_t>(nvs));
  a.hwd = FastDiv(static_cast<uint32_t>(p.size2));
  a.rpi = static_cast<uint32_t>(rpi);
  a.active = static_cast<uint32_t>(rpi * nvs);
  const int64_t packs = p.C / G;
  a.per_xcd = (packs % 8 == 0 && tune_int("BN_PACK_XCD_MAP", 1)) ? static_cast<uint32_t>(packs / 8) : 0u;
  a.row_stride = static_cast<uint32_t>(p.C * p.size2);
  a.edge_lines = (p.C * p.size2 * esz) % 128 == 0 && tune_int("BN_PACK_EDGE_STORES", 1);
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  a.inv_N = static_cast<float>(1.0 / N);
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  (void)vec;
  return true;
}

} // namespace

bool bn_pack_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnPackArgs a;
  int nl = 0;
  if (!p.out || !pack_args(p, false, a, nl)) return false;
  a.y = p.out;
  a.beta = p.beta;
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  const unsigned grid = a.C / a.G;
  *status = p.dtype == NBLAHIP_F16 ? run_pack_fwd<__half, 8>(nl, a, grid, st)
                                   : run_pack_fwd<float, 4>(nl, a, grid, st);
  return true;
}

bool bn_pack_bwd(const BnProblem &p, hipStream_t st, int *status) {
  BnPackArgs a;
  int nl = 0;
  if (!p.batch_stat || (!p.out && !p.dgamma && !p.dbeta)) return false;
  if (!pack_args(p, true, a, nl)) return false;
  a.dy = p.dy;
  a.dx = p.out;
  a.mean = const_cast<float *>(p.mean);
  a.var = const_cast<float *>(p.var);
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.dgamma = p.dgamma;
  a.dbeta = p.dbeta;
  a.accum_dx = p.accum_dx;
  a.accum_g = p.accum_g;
  a.accum_b = p.accum_b;
  const unsigned grid = a.C / a.G;
  *status = p.dtype == NBLAHIP_F16 ? run_pack_bwd<__half, 8>(nl, a, grid, st)
                                   : run_pack_bwd<float, 4>(nl, a, grid, st);
  return true;
}

} // namespace nblahip
