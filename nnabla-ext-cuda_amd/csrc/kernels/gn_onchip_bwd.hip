// GroupNormalization backward for groups of 64 KB - 336 KB (channel-first),
// with the group held on one CU.
//
// The row kernels (rows.cuh) keep a group's x and dy in 8 vectors per thread of
// a 1024-thread block: 128 KB.  Beyond that the backward streams: the
// per-plane sums in one pass, dx in a second (5 S).  Here one 1024-thread block
// per group holds up to 21 vectors of x per thread (12 in registers, 9 in LDS)
// and parks dy in the LDS that x leaves free (9 slots of 16 KB in all; the
// vectors of dy beyond them are read again for dx): 3 S for groups of up to
// 144 KB, 3.5 S at 336 KB.
//
// With xh = (x-mean)*istd and g_c the channel's gamma, per group:
//   s1 = sum g_c*dy, t2 = sum g_c*dy*xh,
//   cA = -istd*t2/R + 2*dvar*std/R,  cb = -s1*istd/R + dmean/R,
//   dx = g_c*istd*dy + cA*xh + cb
// (kernel/group_normalization.cuh:117-206 of the reference).  A plane is a
// whole number of 64-vector runs, so a wave's load lies inside one channel and
// the per-channel (sum dy*xh, sum dy) the parameter gradients need are wave
// sums, recorded per run and added per channel in run order; they go to the
// workspace as [row][channel of the group][2] for the batch sum that follows.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"

namespace nblahip {

namespace {

constexpr int kGnOnchipMaxCpg = 128;

struct GnOnchipArgs {
  const void *x, *dy;
  void *dx; // may be null
  const float *gamma;
  const float *mean, *var, *dmean, *dvar;
  float *pairs;  // [rows][cpg][2]
  uint32_t G;    // groups per sample (gamma of row r starts at (r % G) * cpg)
  uint32_t cpg;  // channels per group
  uint32_t nv;   // vectors per row
  FastDiv rpc;   // 64-vector runs per channel (planes of whole runs)
  FastDiv pv;    // vectors per plane (planes of 8, 16 or 32 vectors: SUB > 0)
  float eps, inv_R, one;
  int accum_dx;
};

} // namespace

// SUB > 0: planes of 64 >> SUB vectors, i.e. 2, 4 or 8 channels side by side
// in a wave's load; the per-channel sums are sums over the lanes of a channel.
template <typename T, int VEC, int NL, int NXS, int ND, int B, int SUB = 0>
__global__ void __launch_bounds__(kOnchipBlock)
gn_onchip_bwd_kernel(const GnOnchipArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  static_assert(NXS + ND <= 9 && NXS < NL, "LDS slots");
  constexpr int NXR = NL - NXS;
  constexpr int NW = kOnchipBlock / kWave;
  __shared__ uint4 park[ND > 0 ? ND * kOnchipBlock : 1];
  __shared__ uint4 xlds[NXS > 0 ? NXS * kOnchipBlock : 1];
  // (sum dy*xh, sum dy) per run of 64 vectors; SUB > 0: per channel
  __shared__ float part[SUB > 0 ? 2 * kGnOnchipMaxCpg : 2 * NL * NW];
  __shared__ float gch[kGnOnchipMaxCpg];
  __shared__ float red[32];
  const uint32_t t = threadIdx.x;
  const uint32_t row = blockIdx.x;
  const uint32_t wave = t / kWave, lane = t % kWave;
  const size_t base = static_cast<size_t>(row) * a.nv * VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + base;
  T *__restrict__ dx = a.dx ? static_cast<T *>(a.dx) + base : nullptr;
  // The small loads first, so that they travel with the tensor's.
  const float mean = a.mean[row];
  const float vpe = a.var[row] + a.eps;
  const float p_dvar = a.dvar ? a.dvar[row] : 0.f;
  const float p_dmean = a.dmean ? a.dmean[row] : 0.f;
  const uint32_t pbase = (row % a.G) * a.cpg;
  float g_t = 1.f;
  if (t < a.cpg && a.gamma) g_t = a.gamma[pbase + t];
  const uint32_t last = a.nv - 1u;

  RawVec<T, VEC> xr[NXR];
  {
    RawVec<T, VEC> xp[NXS > 0 ? NXS : 1];
#pragma unroll
    for (int k = 0; k < NXS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NXR + k) * kOnchipBlock + t;
      xp[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NXR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
      xr[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NXS; ++k) xlds[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, xp[k]);
  }
  // (each thread reads back only what it wrote: no barrier)
  auto xvec = [&](int k) -> RawVec<T, VEC> {
    if (k < NXR) return xr[k < NXR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, xlds[(k - NXR) * kOnchipBlock + t]);
  };
  if (t < a.cpg) gch[t] = g_t; // (read behind the barrier that follows pass 1)
  const float istd = 1.0f / sqrtf(vpe);
  const float nmi = -mean * istd;

  // ---- pass 1: (sum dy*xh, sum dy) of every run of 64 vectors
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
        d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(v, last)) * VEC);
      }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        if (k < ND) park[(k < ND ? k : 0) * kOnchipBlock + t] = __builtin_bit_cast(uint4, d[i]);
        float sdx = 0.f, sdy = 0.f;
        if (static_cast<uint32_t>(k) * kOnchipBlock + t < a.nv) {
          const RawVec<T, VEC> xk = xvec(k);
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float xh = norm_elem<T, VEC>(xk, j, mean, istd, nmi);
            sdx = elem_fma<T, VEC>(d[i], j, xh, sdx);
            sdy = elem_fma<T, VEC>(d[i], j, a.one, sdy);
          }
        }
        if constexpr (SUB > 0) {
          constexpr int PV = kWave >> SUB;
          sdx = group_sum<PV>(sdx);
          sdy = group_sum<PV>(sdy);
          const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
          if (lane % PV == 0 && v < a.nv) { // (a channel lies in one wave's load: written once)
            part[2 * (v / PV)] = sdx;
            part[2 * (v / PV) + 1] = sdy;
          }
        } else {
          sdx = wave_sum(sdx);
          sdy = wave_sum(sdy);
          if (lane == 0) {
            part[2 * (k * NW + wave)] = sdx;
            part[2 * (k * NW + wave) + 1] = sdy;
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0); // the next batch's loads stay below: hoisted, the batches add up
  }
  lds_barrier();
  // Channel c owns the runs [c*rpc, (c+1)*rpc); its pair goes to the workspace,
  // and with gamma into the group's (s1, t2).
  float c1 = 0.f, c2 = 0.f;
  if (t < a.cpg) {
    float sdx = 0.f, sdy = 0.f;
    if constexpr (SUB > 0) {
      sdx = part[2 * t];
      sdy = part[2 * t + 1];
    } else {
      for (uint32_t e = t * a.rpc.d; e < (t + 1u) * a.rpc.d; ++e) {
        sdx += part[2 * e];
        sdy += part[2 * e + 1];
      }
    }
    if (a.pairs) {
      const size_t o = 2 * (static_cast<size_t>(row) * a.cpg + t);
      a.pairs[o] = sdx;
      a.pairs[o + 1] = sdy;
    }
    c1 = g_t * sdy;
    c2 = g_t * sdx;
  }
  c1 = onchip_block_sum(c1, red);
  c2 = onchip_block_sum(c2, red);
  if (dx == nullptr) return;

  // ---- pass 2: dx = dy*g_c*istd + xh*cA + cb  (half: x*A2 + B2, one mixed fma)
#pragma unroll
  for (int k = 0; k < NXR; ++k) forget<T, VEC>(xr[k]);
  const float cA = -istd * c2 * a.inv_R + (a.dvar ? 2.f * p_dvar * (vpe * istd) * a.inv_R : 0.f);
  const float cb = -c1 * istd * a.inv_R + (a.dmean ? p_dmean * a.inv_R : 0.f);
  const float A2 = istd * cA;
  const float B2 = sizeof(T) == 2 ? fmaf(nmi, cA, cb) : cb;
  auto emit = [&](const RawVec<T, VEC> &xv, const RawVec<T, VEC> &dv, int k, uint32_t v) {
    const float gi = (SUB > 0 ? gch[v >> (6 - SUB)] : gch[a.rpc.div(static_cast<uint32_t>(k) * NW + wave)]) * istd;
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float xt;
      if constexpr (sizeof(T) == 2) {
        xt = elem_fma<T, VEC>(xv, j, A2, B2);
      } else {
        xt = fmaf(elem_fma<T, VEC>(xv, j, a.one, -mean), A2, B2);
      }
      o[j] = elem_fma<T, VEC>(dv, j, gi, xt);
    }
    T *dst = dx + static_cast<size_t>(v) * VEC;
    if (a.accum_dx) {
      float old[VEC];
      load_vec<T, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] += old[j];
    }
    store_vec<T, VEC>(dst, o);
  };
  const uint32_t t2 = fresh(t);
#pragma unroll
  for (int k = 0; k < ND && k < NL; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
    if (v < a.nv) emit(xvec(k), __builtin_bit_cast(RawVec<T, VEC>, park[k * kOnchipBlock + t]), k, v);
  }
  float lastv = B2;
#pragma unroll
  for (int k0 = ND; k0 < NL; k0 += B) {
    const uint32_t t3 = fresh_after(t, lastv);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t3;
        d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(v, last)) * VEC);
      }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t3;
      if (k < NL && v < a.nv) {
        emit(xvec(k < NL ? k : 0), d[i], k, v);
        lastv = __builtin_bit_cast(float, __builtin_bit_cast(uint4, d[i]).x);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

namespace {

template <typename T, int VEC, int SUB>
int run_gn_onchip_bwd(int nl, const GnOnchipArgs &a, unsigned grid, hipStream_t st) {
  constexpr int kB = sizeof(T) == 2 ? 2 : 4;
#define GN_CASE(NL, NXS, ND)                                                                     \
  if (nl <= (NL)) {                                                                              \
    NBLAHIP_LAUNCH("gn_onchip_bwd_kernel", (gn_onchip_bwd_kernel<T, VEC, NL, NXS, ND, kB, SUB>), \
                   dim3(grid), dim3(kOnchipBlock), 0, st, a);                                    \
    return last_launch_status();                                                                 \
  }
  GN_CASE(2, 0, 2)
  GN_CASE(3, 0, 3)
  GN_CASE(5, 0, 5)
  GN_CASE(7, 0, 7)
  GN_CASE(9, 0, 9)
  GN_CASE(12, 0, 9)
  if constexpr (SUB == 0) {
    GN_CASE(14, 2, 7)
    GN_CASE(16, 4, 5)
    GN_CASE(18, 6, 3)
    GN_CASE(21, 9, 0)
  }
#undef GN_CASE
  return NBLAHIP_EINVAL;
}

template <typename T, int VEC>
int run_gn_onchip_bwd_sub(int sub, int nl, const GnOnchipArgs &a, unsigned grid, hipStream_t st) {
  switch (sub) {
  case 0: return run_gn_onchip_bwd<T, VEC, 0>(nl, a, grid, st);
  case 1: return run_gn_onchip_bwd<T, VEC, 1>(nl, a, grid, st);
  case 2: return run_gn_onchip_bwd<T, VEC, 2>(nl, a, grid, st);
  default: return run_gn_onchip_bwd<T, VEC, 3>(nl, a, grid, st);
  }
}

} // namespace

// Leaves the per-(sample, channel) pairs in p.ws for the batch sum, as the row
// kernels do.  false: not taken.
bool gn_onchip_bwd(const RowProblem &p, hipStream_t st, int *status) {
  if (!tune_int("GN_ONCHIP_BWD", 1) || p.mode != kRowGN) return false;
  if (!p.out && !p.dgamma && !p.dbeta) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (!aligned16(p.x) || !aligned16(p.dy) || (p.out && !aligned16(p.out))) return false;
  const int64_t cpg = p.channels / p.groups;
  // a wave's load inside one channel (planes of whole 64-vector runs), or 2, 4
  // or 8 whole channels inside a wave's load (planes of 32, 16 or 8 vectors)
  if (p.spatial % vec != 0 || cpg > kGnOnchipMaxCpg) return false;
  const int64_t pv = p.spatial / vec;
  int sub = 0;
  if (pv % 64 != 0) {
    if (pv != 32 && pv != 16 && pv != 8) return false;
    sub = pv == 32 ? 1 : pv == 16 ? 2 : 3;
  }
  const int64_t nv = p.R / vec;
  const int64_t nl = (nv + kOnchipBlock - 1) / kOnchipBlock;
  // Small planes leave half and more of the row kernels' lanes idle (a wave's
  // load there never crosses a channel): from 2 vectors per thread
  // ([16,2560,16,16] half 32.0 us with them).
  if (sub > 0 && (nl < tune_int("GN_ONCHIP_BWD_SMALL_PLANES_MIN_NL", 2) || nl > 12)) return false;
  // From 5 vectors per thread (groups beyond 64 KB), where it also beats the
  // row kernels that hold such a group in 8 vectors per thread of smaller
  // blocks: 80 KB half groups 35.7 -> 26.8 us, 128 KB 26.1 -> 20.4 us, float
  // 128 KB 40.1 -> 37.2 us; at 64 KB ([16,256,64,64] half, two 512-thread
  // blocks per CU there) 20.4 against 22.7 us.
  if (sub == 0 && (nl < tune_int("GN_ONCHIP_BWD_MIN_NL", 5) || nl > 21)) return false;
  // a block is alone on its CU: groups for at least this share of the CUs
  if (p.rows * 100 < static_cast<int64_t>(device_cus()) * tune_int("ROW_ONCHIP_BWD_MIN_PCT", 25))
    return false;
  const bool need_pairs = p.dgamma || p.dbeta;
  if (need_pairs && static_cast<size_t>(p.rows) * cpg * 2 * sizeof(float) > p.ws_bytes) return false;
  GnOnchipArgs a{};
  a.x = p.x;
  a.dy = p.dy;
  a.dx = p.out;
  a.gamma = p.gamma;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.pairs = need_pairs ? static_cast<float *>(p.ws) : nullptr;
  a.G = static_cast<uint32_t>(p.groups);
  a.cpg = static_cast<uint32_t>(cpg);
  a.nv = static_cast<uint32_t>(nv);
  a.rpc = FastDiv(static_cast<uint32_t>(std::max<int64_t>(1, pv / 64)));
  a.pv = FastDiv(static_cast<uint32_t>(pv));
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / static_cast<double>(p.R));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  const unsigned grid = static_cast<unsigned>(p.rows);
  *status = p.dtype == NBLAHIP_F16 ? run_gn_onchip_bwd_sub<__half, 8>(sub, static_cast<int>(nl), a, grid, st)
                                   : run_gn_onchip_bwd_sub<float, 4>(sub, static_cast<int>(nl), a, grid, st);
  return true;
}

} // namespace nblahip
