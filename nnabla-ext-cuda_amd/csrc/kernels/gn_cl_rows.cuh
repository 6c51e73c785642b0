// Channel-last GroupNormalization with the group cached in registers: one
// pass over HBM per direction, like the channel-first row kernels of rows.cuh.
//
// x is [N][P][C] (P spatial positions).  The reduction unit (n, g) is the
// strided tile of P positions x cpg adjacent channels; with cpg a multiple of
// the vector width a thread's vector holds VEC channels of one position, and
// because cvg = cpg / VEC divides the block size a thread always meets the
// same VEC channels: their gamma/beta (and, backward, their dgamma/dbeta
// partial sums) live in registers.
//
// A vector is 16 bytes of a 128-byte line that the neighbouring groups of the
// same position fill: gpl = 128 B / (cpg * sizeof(T)) groups share every line.
// Workgroups are handed to the 8 XCDs round-robin by linear index, so the block
// index is decoded such that the gpl blocks that share lines are neighbours on
// ONE XCD: its L2 then fetches each line from memory once instead of gpl times
// (one fetch per XCD that holds a sharer).
#pragma once

#include "common.cuh"
#include "launch.hpp"

namespace nblahip {

struct GnClArgs {
  const void *x;
  const void *dy;     // backward only
  void *out;          // y (forward) or dx (backward, may be null)
  const float *gamma; // [C], may be null
  const float *beta;  // [C], may be null (forward only)
  float *mean;        // [N*G] forward: written; backward: read
  float *var;
  const float *dmean; // may be null
  const float *dvar;  // may be null
  float *pairs;       // backward: [N][C][2] = (sum dy*xh, sum dy) per sample and channel
  int P, C, G, cpg;
  int units;          // N * G
  FastDiv cvg;        // channel vectors per group (cpg / VEC); divides the block size
  int gpl;            // groups sharing a cache line, 1: plain block order
  float eps, inv_R, one;
  int accum_dx;
  // BatchNormalization [M, C] through the instance kernels (one "sample" of M
  // positions): running statistics of the forward, and dgamma/dbeta written
  // by the backward itself (there is no batch to sum over; pairs unused).
  float *rmean, *rvar;
  float decay, unbias;
  float *dgamma, *dbeta;
  int accum_g, accum_b;
  int direct_params;
  // FusedBatchNormalization through the same kernels: forward
  // y = max(0, bn(x) [+ z]); backward dy is first gated by y > 0 and the gated
  // dy is the gradient of z (dz, optional).
  const void *z;
  const void *y;
  void *dz;
  int accum_dz;
  // Wide forward kernels (a block takes several neighbouring groups / channel
  // vectors): G counts the blocks per sample there, groups the real groups
  // per sample, chunk the vectors a block covers per position.
  int groups;
  FastDiv chunk;
};

constexpr int kXcds = 8;

// Unit (n*G + g) of this block, or -1 for the padding blocks of the XCD map:
// block b runs on XCD b % 8; consecutive blocks of one XCD take the gpl
// members of one line-sharing set, then the next set of that XCD.
__device__ __forceinline__ int gn_cl_unit(const GnClArgs &a) {
  const uint32_t b = blockIdx.x;
  if (a.gpl <= 1) return static_cast<int>(b);
  const uint32_t xcd = b % kXcds, r = b / kXcds;
  const uint32_t m = r % a.gpl, set = (r / a.gpl) * kXcds + xcd;
  const uint32_t unit = set * a.gpl + m;
  return unit < static_cast<uint32_t>(a.units) ? static_cast<int>(unit) : -1;
}

template <int TPR> __device__ __forceinline__ float gn_cl_block_sum(float v, float *lds) {
  v = wave_sum(v);
  constexpr int NW = TPR / kWave;
  const int wave = threadIdx.x / kWave;
  lds_barrier();
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  lds_barrier();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) total += lds[i];
  return total;
}

// ---------------------------------------------------------------------------
// Forward.  Block = one (n, g); thread t owns channel vector t % cvg and the
// positions t / cvg + k * (TPR / cvg), k < NL.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(TPR)
gn_cl_row_fwd_kernel(const GnClArgs a) {
  __shared__ float lds[TPR / kWave];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, g = static_cast<uint32_t>(unit) % a.G;
  const uint32_t pos0 = a.cvg.div(threadIdx.x);
  const uint32_t cv = threadIdx.x - pos0 * a.cvg.d;
  const uint32_t pstep = TPR / a.cvg.d;
  const uint32_t ch = g * a.cpg + cv * VEC; // first of this thread's channels
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(n) * a.P * a.C + ch;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(n) * a.P * a.C + ch;

  RawVec<T, VEC> raw[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    raw[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + static_cast<size_t>(ok ? pos : 0u) * a.C));
  }
  float gam[VEC], bet[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    gam[j] = a.gamma ? a.gamma[ch + j] : 1.f;
    bet[j] = a.beta ? a.beta[ch + j] : 0.f;
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
  const float mean = gn_cl_block_sum<TPR>(s, lds) * a.inv_R;
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (pos0 + k * pstep < static_cast<uint32_t>(a.P)) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
        q = fmaf(d, d, q);
      }
    }
  }
  const float var = gn_cl_block_sum<TPR>(q, lds) * a.inv_R;
  const float istd = inv_std(var, a.eps);
  if (threadIdx.x == 0) {
    a.mean[unit] = mean;
    a.var[unit] = var;
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float sc[VEC], sh[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    sc[j] = gam[j] * istd;
    sh[j] = fmaf(-mean, sc[j], bet[j]); // half output: x*sc + sh in one mixed fma
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(raw[k], j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), sc[j], bet[j]);
        }
      }
      store_vec<T, VEC, false>(y + static_cast<size_t>(pos) * a.C, o);
    }
  }
}

// ---------------------------------------------------------------------------
// Backward: dx and the per-(n, channel) pairs behind dgamma/dbeta.  With
// xh = (x-mean)*istd and dg = dy*gamma:
//   s1 = sum dg, t2 = sum dg*xh, cA = -istd*t2/R + 2*dvar*std/R,
//   cb = -s1*istd/R + dmean/R, dx = dg*istd + cA*xh + cb
// (the algebra of the channel-first row kernel).  A thread's channels are
// fixed, so its VEC pairs (sum dy*xh, sum dy) accumulate in registers; threads
// with the same channel vector are folded by wave sums and an LDS pass.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(TPR, (TPR == 512 ? 4 : 1))
gn_cl_row_bwd_kernel(const GnClArgs a) {
  constexpr int NW = TPR / kWave;
  __shared__ float fold[NW][2 * VEC * 8]; // per wave: up to 8 channel vectors x 2*VEC sums
  __shared__ float chs[2 * VEC * 8];      // folded per-channel sums of the group (cpg <= 8*VEC)
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, g = static_cast<uint32_t>(unit) % a.G;
  const uint32_t pos0 = a.cvg.div(threadIdx.x);
  const uint32_t cv = threadIdx.x - pos0 * a.cvg.d;
  const uint32_t pstep = TPR / a.cvg.d;
  const uint32_t ch = g * a.cpg + cv * VEC;
  const size_t slab = static_cast<size_t>(n) * a.P * a.C + ch;
  const T *__restrict__ x = static_cast<const T *>(a.x) + slab;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + slab;
  T *__restrict__ dx = a.out ? static_cast<T *>(a.out) + slab : nullptr;

  RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    const size_t off = static_cast<size_t>(ok ? pos : 0u) * a.C;
    xr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + off));
    dr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + off));
  }
  float gam[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) gam[j] = a.gamma ? a.gamma[ch + j] : 1.f;
  const float mean = a.mean[unit];
  const float vpe = a.var[unit] + a.eps;
  const float istd = 1.0f / sqrtf(vpe);
  const float nmi = -mean * istd;

  // per-channel partial sums of this thread (padded positions hold dy = 0)
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
      sdx[j] = elem_fma<T, VEC>(dr[k], j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dr[k], j, a.one, sdy[j]);
    }
  }
  // Lanes with equal lane % cvg share channels (cvg is a power of two <= 8):
  // butterfly over the lane bits above log2(cvg), then one LDS row per wave.
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  // (through the LDS crossbar: on the vector unit's swap paths, xor_add, these
  // two kernels need a few registers more than their 128 and spill)
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    for (int off = static_cast<int>(a.cvg.d); off < kWave; off <<= 1) {
      sdx[j] += __shfl_xor(sdx[j], off);
      sdy[j] += __shfl_xor(sdy[j], off);
    }
  }
  if (lane < static_cast<int>(a.cvg.d)) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      fold[wave][(lane * VEC + j) * 2] = sdx[j];
      fold[wave][(lane * VEC + j) * 2 + 1] = sdy[j];
    }
  }
  lds_barrier();
  for (int e = threadIdx.x; e < 2 * a.cpg; e += TPR) { // up to 128 entries, 64 threads and more
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w][e];
    chs[e] = t;
    // entry 2*c of the group is (sum dy*xh) of its channel c, 2*c+1 (sum dy)
    a.pairs[2 * (static_cast<size_t>(n) * a.C + g * a.cpg) + e] = t;
  }
  lds_barrier();
  float s1 = 0.f, t2 = 0.f;
  for (int c = 0; c < a.cpg; ++c) {
    const float gc = a.gamma ? a.gamma[g * a.cpg + c] : 1.f;
    t2 = fmaf(gc, chs[2 * c], t2);
    s1 = fmaf(gc, chs[2 * c + 1], s1);
  }
  if (dx == nullptr) return;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    keep_packed<T, VEC>(xr[k]);
    keep_packed<T, VEC>(dr[k]);
  }
  const float cA = -istd * t2 * a.inv_R + (a.dvar ? 2.f * a.dvar[unit] * (vpe * istd) * a.inv_R : 0.f);
  const float cb = -s1 * istd * a.inv_R + (a.dmean ? a.dmean[unit] * a.inv_R : 0.f);
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        o[j] = elem_fma<T, VEC>(dr[k], j, gam[j] * istd, fmaf(xh, cA, cb));
      }
      T *p = dx + static_cast<size_t>(pos) * a.C;
      if (a.accum_dx) {
        float old[VEC];
        load_vec<T, VEC>(p, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] += old[j];
      }
      store_vec<T, VEC, false>(p, o);
    }
  }
}

// ---------------------------------------------------------------------------
// Channel-last InstanceNormalization with the instances cached in registers.
// A block owns sample n and one channel vector (VEC adjacent channels, i.e.
// VEC instances): thread t holds positions t + k*TPR, its vector element j
// always belongs to channel ch + j, so the statistics are VEC sums per thread,
// folded over the block (wave sums, then LDS).  GnClArgs as above with
// G = C / VEC "groups", cpg = VEC, cvg = 1; mean/var/dmean/dvar are indexed
// n*C + channel.  The block order shares cache lines between neighbouring
// channel vectors exactly as for the groups.
// ---------------------------------------------------------------------------
template <int TPR, int VEC>
__device__ __forceinline__ void in_cl_block_sums(float (&v)[VEC], float (*lds)[VEC]) {
  constexpr int NW = TPR / kWave;
  const int wave = threadIdx.x / kWave;
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = wave_sum(v[j]);
  lds_barrier(); // previous readers of lds are done
  if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) lds[wave][j] = v[j];
  }
  lds_barrier();
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += lds[w][j];
    v[j] = t;
  }
}

// FUSE: 0 plain, 1 y = max(0, .), 2 y = max(0, . + z).
template <typename T, int VEC, int NL, int TPR, int FUSE = 0>
__global__ void __launch_bounds__(TPR)
in_cl_row_fwd_kernel(const GnClArgs a) {
  __shared__ float lds[TPR / kWave][VEC];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, cv = static_cast<uint32_t>(unit) % a.G;
  const uint32_t ch = cv * VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(n) * a.P * a.C + ch;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(n) * a.P * a.C + ch;

  RawVec<T, VEC> raw[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = threadIdx.x + k * TPR;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    raw[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + static_cast<size_t>(ok ? pos : 0u) * a.C));
  }
  float gam[VEC], bet[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    gam[j] = a.gamma ? a.gamma[ch + j] : 1.f;
    bet[j] = a.beta ? a.beta[ch + j] : 0.f;
  }
  float mean[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) mean[j] = elem_fma<T, VEC>(raw[k], j, a.one, mean[j]);
  }
  in_cl_block_sums<TPR, VEC>(mean, lds);
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] *= a.inv_R;
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float var[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) var[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (threadIdx.x + k * TPR < static_cast<uint32_t>(a.P)) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean[j]);
        var[j] = fmaf(d, d, var[j]);
      }
    }
  }
  in_cl_block_sums<TPR, VEC>(var, lds);
  float sc[VEC], sh[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    var[j] *= a.inv_R;
    sc[j] = gam[j] * inv_std(var[j], a.eps);
    sh[j] = fmaf(-mean[j], sc[j], bet[j]);
  }
  if (threadIdx.x < VEC) {
    // lane j publishes channel j (every lane holds all VEC values)
    float m = mean[0], v = var[0];
#pragma unroll
    for (int j = 1; j < VEC; ++j) {
      m = threadIdx.x == j ? mean[j] : m;
      v = threadIdx.x == j ? var[j] : v;
    }
    const size_t c = static_cast<size_t>(n) * a.C + ch + threadIdx.x;
    a.mean[c] = m;
    a.var[c] = v;
    if (a.rmean) a.rmean[c] = a.decay * a.rmean[c] + (1.f - a.decay) * m;
    if (a.rvar) a.rvar[c] = a.decay * a.rvar[c] + (1.f - a.decay) * v * a.unbias;
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = threadIdx.x + k * TPR;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(raw[k], j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean[j]), sc[j], bet[j]);
        }
      }
      if constexpr (FUSE == 2) {
        const T *zp = static_cast<const T *>(a.z) + static_cast<size_t>(n) * a.P * a.C + ch;
        const RawVec<T, VEC> zr = load_raw<T, VEC>(zp + static_cast<size_t>(pos) * a.C);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = elem_fma<T, VEC>(zr, j, a.one, o[j]);
      }
      if constexpr (FUSE != 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = fmaxf(0.f, o[j]);
      }
      store_vec<T, VEC, false>(y + static_cast<size_t>(pos) * a.C, o);
    }
  }
}

// Backward, per channel c of the block: sdx = sum dy*xh, sdy = sum dy (also the
// pair behind dgamma/dbeta), dx = g*istd*dy + cA*xh + cb with
// cA = -istd*g*sdx/P + 2*dvar*std/P, cb = -g*sdy*istd/P + dmean/P.
// FUSED: dy := dy where y > 0 else 0 first; dz (optional) receives it.
template <typename T, int VEC, int NL, int TPR, bool FUSED = false>
__global__ void __launch_bounds__(TPR, (TPR == 512 ? 4 : 1))
in_cl_row_bwd_kernel(const GnClArgs a) {
  __shared__ float lds[TPR / kWave][VEC];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, cv = static_cast<uint32_t>(unit) % a.G;
  const uint32_t ch = cv * VEC;
  const size_t slab = static_cast<size_t>(n) * a.P * a.C + ch;
  const size_t stat = static_cast<size_t>(n) * a.C + ch;
  const T *__restrict__ x = static_cast<const T *>(a.x) + slab;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + slab;
  T *__restrict__ dx = a.out ? static_cast<T *>(a.out) + slab : nullptr;

  RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = threadIdx.x + k * TPR;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    const size_t off = static_cast<size_t>(ok ? pos : 0u) * a.C;
    xr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + off));
    dr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + off));
    if constexpr (FUSED) {
      const RawVec<T, VEC> yr = load_raw<T, VEC>(static_cast<const T *>(a.y) + slab + off);
      dr[k] = raw_relu_mask<T, VEC>(dr[k], yr);
      if (a.dz && ok) {
        T *dzp = static_cast<T *>(a.dz) + slab + off;
        if (a.accum_dz) {
          float g[VEC], old[VEC];
          unpack<T, VEC>(dr[k], g);
          load_vec<T, VEC>(dzp, old);
#pragma unroll
          for (int j = 0; j < VEC; ++j) g[j] += old[j];
          store_vec<T, VEC, false>(dzp, g);
        } else {
          store_raw<T, VEC, false>(dzp, dr[k]);
        }
      }
    }
  }
  float istd[VEC], nmi[VEC], mean[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mean[j] = a.mean[stat + j];
    istd[j] = 1.0f / sqrtf(a.var[stat + j] + a.eps);
    nmi[j] = -mean[j] * istd[j];
  }
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr[k], j, mean[j], istd[j], nmi[j]);
      sdx[j] = elem_fma<T, VEC>(dr[k], j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dr[k], j, a.one, sdy[j]);
    }
  }
  in_cl_block_sums<TPR, VEC>(sdx, lds);
  in_cl_block_sums<TPR, VEC>(sdy, lds);
  if (threadIdx.x < VEC) {
    float px = sdx[0], py = sdy[0];
#pragma unroll
    for (int j = 1; j < VEC; ++j) {
      px = threadIdx.x == j ? sdx[j] : px;
      py = threadIdx.x == j ? sdy[j] : py;
    }
    const size_t c = stat + threadIdx.x;
    if (a.direct_params) {
      if (a.dgamma) a.dgamma[c] = px + (a.accum_g ? a.dgamma[c] : 0.f);
      if (a.dbeta) a.dbeta[c] = py + (a.accum_b ? a.dbeta[c] : 0.f);
    } else {
      a.pairs[2 * c] = px;
      a.pairs[2 * c + 1] = py;
    }
  }
  if (dx == nullptr) return;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    keep_packed<T, VEC>(xr[k]);
    keep_packed<T, VEC>(dr[k]);
  }
  float gi[VEC], cA[VEC], cb[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const float g = a.gamma ? a.gamma[ch + j] : 1.f;
    const float vpe = a.var[stat + j] + a.eps;
    gi[j] = g * istd[j];
    cA[j] = -istd[j] * g * sdx[j] * a.inv_R +
            (a.dvar ? 2.f * a.dvar[stat + j] * (vpe * istd[j]) * a.inv_R : 0.f);
    cb[j] = -g * sdy[j] * istd[j] * a.inv_R + (a.dmean ? a.dmean[stat + j] * a.inv_R : 0.f);
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = threadIdx.x + k * TPR;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean[j], istd[j], nmi[j]);
        o[j] = elem_fma<T, VEC>(dr[k], j, gi[j], fmaf(xh, cA[j], cb[j]));
      }
      T *p = dx + static_cast<size_t>(pos) * a.C;
      if (a.accum_dx) {
        float old[VEC];
        load_vec<T, VEC>(p, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] += old[j];
      }
      store_vec<T, VEC, false>(p, o);
    }
  }
}

// ---------------------------------------------------------------------------
// Wide forward kernels.  A 16-byte vector is an eighth of the 128-byte line
// that L2 hands to the CU: with one group (or channel vector) per block every
// line crosses that path once per sharer, and the forward runs at the rate of
// that path, not of HBM (the same 33 MB tensor: 24 us at 16-byte pieces per
// position, 17 us at 32, 13.5 us at 64).  Here a block takes GPB neighbouring
// groups (CVB channel vectors): its threads read 32- or 64-byte pieces.  The
// statistics stay per group (per channel), so the block sums are segmented:
// a butterfly over the lanes that hold the same piece of the chunk, then LDS.
// ---------------------------------------------------------------------------
// PARK: x waits in LDS instead of registers (the 1024 x 8 layout: with 8
// statistics per thread beside 8 vectors of x the registers run out).
template <typename T, int VEC, int NL, int TPR, int CVB, bool PARK = false>
__global__ void __launch_bounds__(TPR)
in_cl_wide_fwd_kernel(const GnClArgs a) {
  static_assert(!PARK || sizeof(RawVec<T, VEC>) == 16, "parked vectors are 16 bytes");
  __shared__ uint4 park[PARK ? NL * TPR : 1];
  constexpr int NW = TPR / kWave;
  constexpr uint32_t PST = TPR / CVB; // positions a block covers per load
  __shared__ float lds[NW][CVB][VEC];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, cb = static_cast<uint32_t>(unit) % a.G;
  const uint32_t cvx = threadIdx.x % CVB, pos0 = threadIdx.x / CVB;
  const uint32_t ch = (cb * CVB + cvx) * VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(n) * a.P * a.C + ch;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(n) * a.P * a.C + ch;

  RawVec<T, VEC> raw[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * PST;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    raw[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + static_cast<size_t>(ok ? pos : 0u) * a.C));
  }
  if constexpr (PARK) {
#pragma unroll
    for (int k = 0; k < NL; ++k) park[k * TPR + threadIdx.x] = __builtin_bit_cast(uint4, raw[k]);
    asm volatile("" ::: "memory"); // read back from LDS from here on
  }
  auto xv = [&](int k) -> RawVec<T, VEC> {
    if constexpr (PARK) {
      return __builtin_bit_cast(RawVec<T, VEC>, park[k * TPR + threadIdx.x]);
    } else {
      return raw[k];
    }
  };
  float gam[VEC], bet[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    gam[j] = a.gamma ? a.gamma[ch + j] : 1.f;
    bet[j] = a.beta ? a.beta[ch + j] : 0.f;
  }
  // sums over the threads with the same channel vector (lane % CVB == cvx)
  auto block_sums = [&](float (&v)[VEC]) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    lanes_sum_from<VEC>(v, static_cast<uint32_t>(CVB));
    lds_barrier(); // previous readers of lds are done
    if (lane < CVB) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) lds[wave][lane][j] = v[j];
    }
    lds_barrier();
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) t += lds[w][cvx][j];
      v[j] = t;
    }
  };
  float mean[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const RawVec<T, VEC> r = xv(k);
#pragma unroll
    for (int j = 0; j < VEC; ++j) mean[j] = elem_fma<T, VEC>(r, j, a.one, mean[j]);
  }
  block_sums(mean);
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] *= a.inv_R;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if constexpr (!PARK) keep_packed<T, VEC>(raw[k]);
  }
  float var[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) var[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (pos0 + k * PST < static_cast<uint32_t>(a.P)) {
      const RawVec<T, VEC> r = xv(k);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = elem_fma<T, VEC>(r, j, a.one, -mean[j]);
        var[j] = fmaf(d, d, var[j]);
      }
    }
  }
  block_sums(var);
  float sc[VEC], sh[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    var[j] *= a.inv_R;
    sc[j] = gam[j] * inv_std(var[j], a.eps);
    sh[j] = fmaf(-mean[j], sc[j], bet[j]);
  }
  if (threadIdx.x < CVB) { // thread t < CVB holds channel vector t of the block
    const size_t c = static_cast<size_t>(n) * a.C + ch;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      a.mean[c + j] = mean[j];
      a.var[c + j] = var[j];
    }
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if constexpr (!PARK) keep_packed<T, VEC>(raw[k]);
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * PST;
    if (pos < static_cast<uint32_t>(a.P)) {
      const RawVec<T, VEC> r = xv(k);
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(r, j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mean[j]), sc[j], bet[j]);
        }
      }
      store_vec<T, VEC, false>(y + static_cast<size_t>(pos) * a.C, o);
    }
  }
}

// GroupNormalization: the chunk of a position holds GPB groups of cvg vectors
// each; thread t owns vector t % chunk of the positions t / chunk + k * (TPR /
// chunk).  Lanes with the same t % chunk are folded first, then the cvg lanes
// of a group (aligned runs of a power of two), then the waves through LDS.
template <typename T, int VEC, int NL, int TPR, int GPB>
__global__ void __launch_bounds__(TPR)
gn_cl_wide_fwd_kernel(const GnClArgs a) {
  constexpr int NW = TPR / kWave;
  __shared__ float lds[NW][GPB];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, gb = static_cast<uint32_t>(unit) % a.G;
  const uint32_t pos0 = a.chunk.div(threadIdx.x);
  const uint32_t cvx = threadIdx.x - pos0 * a.chunk.d;
  const uint32_t sg = a.cvg.div(cvx); // group of the block this thread belongs to
  const uint32_t pstep = TPR / a.chunk.d;
  const uint32_t ch = gb * GPB * a.cpg + cvx * VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(n) * a.P * a.C + ch;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(n) * a.P * a.C + ch;

  RawVec<T, VEC> raw[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    raw[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + static_cast<size_t>(ok ? pos : 0u) * a.C));
  }
  float gam[VEC], bet[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    gam[j] = a.gamma ? a.gamma[ch + j] : 1.f;
    bet[j] = a.beta ? a.beta[ch + j] : 0.f;
  }
  auto group_block_sum = [&](float v) -> float {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    v = lanes_sum_from(v, a.chunk.d);
    v = lanes_sum_below(v, a.cvg.d);
    lds_barrier(); // previous readers of lds are done
    if (lane < static_cast<int>(a.chunk.d) && cvx == sg * a.cvg.d) lds[wave][sg] = v;
    lds_barrier();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += lds[w][sg];
    return t;
  };
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
  const float mean = group_block_sum(s) * a.inv_R;
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (pos0 + k * pstep < static_cast<uint32_t>(a.P)) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
        q = fmaf(d, d, q);
      }
    }
  }
  const float var = group_block_sum(q) * a.inv_R;
  const float istd = inv_std(var, a.eps);
  if (threadIdx.x < a.chunk.d && cvx == sg * a.cvg.d) {
    const uint32_t u = n * static_cast<uint32_t>(a.groups) + gb * GPB + sg;
    a.mean[u] = mean;
    a.var[u] = var;
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float sc[VEC], sh[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    sc[j] = gam[j] * istd;
    sh[j] = fmaf(-mean, sc[j], bet[j]);
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * pstep;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(raw[k], j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), sc[j], bet[j]);
        }
      }
      store_vec<T, VEC, false>(y + static_cast<size_t>(pos) * a.C, o);
    }
  }
}

// Wide backward (half data, 8 channels per group, or instances): a block takes
// GPB neighbouring groups / channel vectors of a sample, keeps x in registers
// and parks dy in LDS (each thread reads back what it wrote), so both tensors
// cross the memory system once, in 32- or 64-byte pieces: one launch, 3 S,
// where planes beyond 2048 positions otherwise take the three-kernel path
// (6 S).  A thread's vector is the 8 channels of one group (INSTANCE: 8
// instances) at one position; per-channel sums fold over the threads with the
// same piece of the chunk.  Algebra as in gn_cl_row_bwd_kernel /
// in_cl_row_bwd_kernel.
template <int NL, int TPR, int GPB, bool INSTANCE>
__global__ void __launch_bounds__(TPR)
cl_wide_bwd_kernel(const GnClArgs a) {
  using T = __half;
  constexpr int VEC = 8;
  constexpr int NW = TPR / kWave;
  constexpr uint32_t PST = TPR / GPB;
  __shared__ uint4 park[NL * TPR];
  __shared__ float fold[NW][GPB][2 * VEC];
  __shared__ float chs[GPB][2 * VEC];
  const int unit = gn_cl_unit(a);
  if (unit < 0) return;
  const uint32_t n = static_cast<uint32_t>(unit) / a.G, gb = static_cast<uint32_t>(unit) % a.G;
  const uint32_t cvx = threadIdx.x % GPB, pos0 = threadIdx.x / GPB;
  const uint32_t ch = (gb * GPB + cvx) * VEC;
  const size_t slab = static_cast<size_t>(n) * a.P * a.C + ch;
  const T *__restrict__ x = static_cast<const T *>(a.x) + slab;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + slab;
  T *__restrict__ dx = a.out ? static_cast<T *>(a.out) + slab : nullptr;

  RawVec<T, VEC> xr[NL];
  {
    RawVec<T, VEC> dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const uint32_t pos = pos0 + k * PST;
      const bool ok = pos < static_cast<uint32_t>(a.P);
      const size_t off = static_cast<size_t>(ok ? pos : 0u) * a.C;
      xr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + off));
      dr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + off)); // padded positions: dy = 0
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) park[k * TPR + threadIdx.x] = dr[k].v;
  }
  asm volatile("" ::: "memory"); // dy is read back from LDS, not kept in registers
  // statistics of this thread's channels: one pair per group, or one per channel
  constexpr int NS = INSTANCE ? VEC : 1;
  const uint32_t stat = INSTANCE ? n * static_cast<uint32_t>(a.C) + ch
                                 : n * static_cast<uint32_t>(a.groups) + gb * GPB + cvx;
  float mean[NS], istd[NS], nmi[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    mean[i] = a.mean[stat + i];
    istd[i] = 1.0f / sqrtf(a.var[stat + i] + a.eps);
    nmi[i] = -mean[i] * istd[i];
  }
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    RawVec<T, VEC> dr;
    dr.v = park[k * TPR + threadIdx.x];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int i = INSTANCE ? j : 0;
      const float xh = norm_elem<T, VEC>(xr[k], j, mean[i], istd[i], nmi[i]);
      sdx[j] = elem_fma<T, VEC>(dr, j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dr, j, a.one, sdy[j]);
    }
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  // (as above: the swap paths cost this kernel registers it does not have)
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
#pragma unroll
    for (int off = GPB; off < kWave; off <<= 1) {
      sdx[j] += __shfl_xor(sdx[j], off);
      sdy[j] += __shfl_xor(sdy[j], off);
    }
  }
  if (lane < GPB) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      fold[wave][lane][2 * j] = sdx[j];
      fold[wave][lane][2 * j + 1] = sdy[j];
    }
  }
  lds_barrier();
  if (threadIdx.x < GPB * 2 * VEC) {
    const int cv = threadIdx.x / (2 * VEC), e = threadIdx.x % (2 * VEC);
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w][cv][e];
    chs[cv][e] = t;
    // entry 2*c is (sum dy*xh) of channel c of the block's chunk, 2*c+1 (sum dy)
    a.pairs[2 * (static_cast<size_t>(n) * a.C + gb * GPB * VEC) + threadIdx.x] = t;
  }
  lds_barrier();
  if (dx == nullptr) return;
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(xr[k]);
  float gi[VEC], cA[NS], cb[NS];
  if constexpr (INSTANCE) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float g = a.gamma ? a.gamma[ch + j] : 1.f;
      const float vpe = a.var[stat + j] + a.eps;
      gi[j] = g * istd[j];
      cA[j] = -istd[j] * g * chs[cvx][2 * j] * a.inv_R +
              (a.dvar ? 2.f * a.dvar[stat + j] * (vpe * istd[j]) * a.inv_R : 0.f);
      cb[j] = -g * chs[cvx][2 * j + 1] * istd[j] * a.inv_R +
              (a.dmean ? a.dmean[stat + j] * a.inv_R : 0.f);
    }
  } else {
    float s1 = 0.f, t2 = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float g = a.gamma ? a.gamma[ch + j] : 1.f;
      gi[j] = g * istd[0];
      t2 = fmaf(g, chs[cvx][2 * j], t2);
      s1 = fmaf(g, chs[cvx][2 * j + 1], s1);
    }
    const float vpe = a.var[stat] + a.eps;
    cA[0] = -istd[0] * t2 * a.inv_R + (a.dvar ? 2.f * a.dvar[stat] * (vpe * istd[0]) * a.inv_R : 0.f);
    cb[0] = -s1 * istd[0] * a.inv_R + (a.dmean ? a.dmean[stat] * a.inv_R : 0.f);
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = pos0 + k * PST;
    if (pos < static_cast<uint32_t>(a.P)) {
      RawVec<T, VEC> dr;
      dr.v = park[k * TPR + threadIdx.x];
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const int i = INSTANCE ? j : 0;
        const float xh = norm_elem<T, VEC>(xr[k], j, mean[i], istd[i], nmi[i]);
        o[j] = elem_fma<T, VEC>(dr, j, gi[j], fmaf(xh, cA[i], cb[i]));
      }
      T *p = dx + static_cast<size_t>(pos) * a.C;
      if (a.accum_dx) {
        float old[VEC];
        load_vec<T, VEC>(p, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] += old[j];
      }
      store_vec<T, VEC, false>(p, o);
    }
  }
}

} // namespace nblahip
