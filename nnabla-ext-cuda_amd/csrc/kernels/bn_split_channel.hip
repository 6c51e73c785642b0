// BatchNormalization training (planes layout) for tensors with fewer channels
// than CUs: a channel is SPLIT over 2, 4 or 8 workgroups, each of which holds
// its share of the channel's samples on its CU, and the workgroups of a channel
// exchange their partial sums.
//
// With one block per channel (bn_onchip.hip) a [32,64,112,112] tensor keeps 64
// of the 256 CUs busy, and its 800 KB channels do not fit a CU anyway.  Here
// block b = c * SP + sp takes the samples [sp * spb, (sp + 1) * spb) of channel
// c - planes that lie C * size2 elements apart, vector v of the block at
// k * 1024 + t as in bn_onchip.hip - reduces them in registers, publishes
// (mean, m2) - backward: (sum dy*xh, sum dy) - as {value, epoch} words
// (xchg.cuh), polls its SP - 1 partners' words, merges all parts in block order
// (every block of a channel arrives at the same bits; block 0 writes the
// statistics) and finishes from registers: x crosses the memory system once,
// 2 S forward.  The backward holds x in registers and parks dy in LDS (the
// vectors beyond what LDS takes are read a second time): 3 S.
//
// Every wait is a bounded poll.  A partner's part that does not turn up is
// computed by the block that needs it, from global memory, in the partner's
// arithmetic (its thread map, its order of additions), so every wave reaches
// the end of the kernel whatever the other blocks do and the result does not
// depend on who computed what.  The blocks of a channel are neighbours in the
// grid: when the grid takes more than one round, a block's partners are
// running or next in line.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"
#include "xchg.cuh"

namespace nblahip {

namespace {

constexpr int kChanSplitMax = 8; // blocks per channel

struct BnChanSplitArgs {
  const void *x;
  void *y;
  const float *gamma, *beta;
  float *mean, *var, *rmean, *rvar;
  uint32_t C, size2;
  uint32_t N;   // samples
  uint32_t SP;  // blocks per channel
  uint32_t spb; // samples per block (the last block of a channel may hold fewer)
  FastDiv vpp;  // vectors per plane
  float inv_N, unbias, decay, eps, one;
  // backward
  const void *dy;
  void *dx;                  // may be null
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;     // may be null
  int accum_dx, accum_g, accum_b;
  unsigned long long *xchg; // [C][SP][2]
  uint32_t epoch;
  int spin;
};

// Samples of block sp of a channel.
__device__ __forceinline__ uint32_t chan_block_samples(const BnChanSplitArgs &a, uint32_t sp) {
  const uint32_t first = sp * a.spb;
  return first >= a.N ? 0u : min(a.spb, a.N - first);
}

// Element offset of vector v of block sp of channel c.
__device__ __forceinline__ uint32_t chan_offset(const BnChanSplitArgs &a, uint32_t c, uint32_t sp,
                                                uint32_t v, int vec) {
  const uint32_t n = a.vpp.div(v);
  const uint32_t w = v - n * a.vpp.d;
  return ((sp * a.spb + n) * a.C + c) * a.size2 + w * static_cast<uint32_t>(vec);
}

// Sum of a and of b over the block, both at once; red: [2][16].
__device__ __forceinline__ void chan_block_sum2(float &a, float &b, float *red) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x / kWave;
  lds_barrier(); // earlier readers of red are done
  if ((threadIdx.x & (kWave - 1)) == 0) {
    red[wave] = a;
    red[16 + wave] = b;
  }
  lds_barrier();
  float ta = 0.f, tb = 0.f;
#pragma unroll
  for (int i = 0; i < kOnchipBlock / kWave; ++i) {
    ta += red[i];
    tb += red[16 + i];
  }
  a = ta;
  b = tb;
}

// (mean, m2) of the samples of block sp of channel c, from global memory, in
// the arithmetic of the block that owns them: a thread's vectors k * 1024 + t
// ascending, s = sum x, the thread's own mean K = s / n, s1 = sum (x - K),
// s2 = sum (x - K)^2, then two block sums.
template <typename T, int VEC>
__device__ __forceinline__ void chan_part_from_memory(const BnChanSplitArgs &a, uint32_t c,
                                                      uint32_t sp, float *red, float &m, float &q) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const uint32_t t = threadIdx.x;
  const uint32_t nvb = chan_block_samples(a, sp) * a.vpp.d;
  float s = 0.f;
#pragma unroll 1
  for (uint32_t v = t; v < nvb; v += kOnchipBlock)
    s = raw_sum<T, VEC>(load_raw<T, VEC>(x + chan_offset(a, c, sp, v, VEC)), s);
  const float nt = t < nvb ? static_cast<float>(((nvb - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
  const float kk = s * (1.0f / fmaxf(nt, 1.f));
  float s1 = 0.f, s2 = 0.f;
#pragma unroll 1
  for (uint32_t v = t; v < nvb; v += kOnchipBlock) {
    const RawVec<T, VEC> r = load_raw<T, VEC>(x + chan_offset(a, c, sp, v, VEC));
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = elem_fma<T, VEC>(r, j, a.one, -kk);
      s1 += d;
      s2 = fmaf(d, d, s2);
    }
  }
  m = onchip_block_sum(s, red) * (1.0f / static_cast<float>(nvb * VEC));
  const float e = kk - m;
  q = onchip_block_sum(fmaf(e, fmaf(nt, e, 2.f * s1), s2), red);
}

// Publishes this block's pair, collects the partners' (thread p polls block p;
// a pair that does not arrive is marked in miss[]).  got: [SP][2].
__device__ __forceinline__ void chan_exchange(const BnChanSplitArgs &a, uint32_t c, uint32_t sp,
                                              float v0, float v1, float *got, int *miss) {
  const uint32_t t = threadIdx.x;
  unsigned long long *slots = a.xchg + static_cast<size_t>(c) * a.SP * 2;
  if (t == 0) {
    xchg_publish(slots + sp * 2, v0, a.epoch);
    xchg_publish(slots + sp * 2 + 1, v1, a.epoch);
    got[2 * sp] = v0;
    got[2 * sp + 1] = v1;
    miss[sp] = 0;
  }
  if (t < a.SP && t != sp) {
    float p0 = 0.f, p1 = 0.f;
    const bool ok = xchg_poll2(slots + t * 2, a.epoch, a.spin, &p0, &p1);
    got[2 * t] = p0;
    got[2 * t + 1] = p1;
    miss[t] = ok ? 0 : 1;
  }
  lds_barrier();
}

// The partners whose pair did not arrive, a bit each: every wave reads the
// flags side by side (one LDS round trip, not one per partner) and gets the
// same mask.  After chan_exchange's barrier.
__device__ __forceinline__ uint64_t chan_missing(const BnChanSplitArgs &a, uint32_t sp, const int *miss) {
  const uint32_t lane = threadIdx.x % kWave;
  return __ballot(lane < a.SP && lane != sp && miss[lane] != 0);
}

} // namespace

template <typename T, int VEC, int NR, int NS>
__global__ void __launch_bounds__(kOnchipBlock)
bn_chan_split_fwd_kernel(const BnChanSplitArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float red[32];
  __shared__ float got[2 * kChanSplitMax];
  __shared__ int miss[kChanSplitMax];
  __shared__ float fin[2];
  const uint32_t t = threadIdx.x;
  const uint32_t c = blockIdx.x / a.SP, sp = blockIdx.x % a.SP;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.y);
  // (asked for now: behind the exchange they would cost a round trip of their own)
  const float gamma_c = a.gamma ? a.gamma[c] : 1.f;
  const float beta_c = a.beta ? a.beta[c] : 0.f;
  const float rmean_c = a.rmean ? a.rmean[c] : 0.f;
  const float rvar_c = a.rvar ? a.rvar[c] : 0.f;
  const uint32_t nvb = chan_block_samples(a, sp) * a.vpp.d;
  const uint32_t last = nvb - 1u;

  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t;
      parked[k] = load_raw<T, VEC>(x + chan_offset(a, c, sp, min(v, last), VEC));
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
      raw[k] = load_raw<T, VEC>(x + chan_offset(a, c, sp, min(v, last), VEC));
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };
  auto held = [&](int k) { return static_cast<int>(t) < static_cast<int>(nvb) - k * kOnchipBlock; };

  // ---- this block's (mean, m2): sums over the thread's own registers as its
  // loads arrive (chan_part_from_memory has the arithmetic, vector by vector
  // in the same order)
  float m, q;
  {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (held(k)) s = raw_sum<T, VEC>(slot(k), s);
    }
    const float nt = t < nvb ? static_cast<float>(((nvb - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
    const float kk = s * (1.0f / fmaxf(nt, 1.f));
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (held(k)) {
        const RawVec<T, VEC> r = slot(k);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(r, j, a.one, -kk);
          s1 += d;
          s2 = fmaf(d, d, s2);
        }
      }
    }
    m = onchip_block_sum(s, red) * (1.0f / static_cast<float>(nvb * VEC));
    const float e = kk - m;
    q = onchip_block_sum(fmaf(e, fmaf(nt, e, 2.f * s1), s2), red);
  }

  // ---- the partners' parts, the merge in block order (Chan), the statistics
  chan_exchange(a, c, sp, m, q, got, miss);
  const uint64_t late = chan_missing(a, sp, miss);
  for (uint64_t todo = late; todo != 0; todo &= todo - 1) {
    const uint32_t p = static_cast<uint32_t>(__builtin_ctzll(todo));
    float pm, pq;
    chan_part_from_memory<T, VEC>(a, c, p, red, pm, pq);
    if (t == 0) {
      got[2 * p] = pm;
      got[2 * p + 1] = pq;
    }
  }
  if (late != 0) lds_barrier();
  if (t == 0) {
    const float per = static_cast<float>(a.vpp.d * VEC);
    float mean = 0.f, m2 = 0.f, n = 0.f;
    for_pairs_in_order(got, 2, static_cast<int>(a.SP), [&](int p, float pm, float pq) {
      const float nb = static_cast<float>(chan_block_samples(a, static_cast<uint32_t>(p))) * per;
      if (p == 0) {
        mean = pm;
        m2 = pq;
        n = nb;
        return;
      }
      const float tot = n + nb;
      const float d = pm - mean;
      const float wgt = nb / tot;
      mean = fmaf(d, wgt, mean);
      m2 = m2 + pq + d * d * (n * wgt);
      n = tot;
    });
    const float var = m2 * a.inv_N;
    fin[0] = mean;
    fin[1] = var;
    if (sp == 0) {
      a.mean[c] = mean;
      a.var[c] = var;
      if (a.rmean) a.rmean[c] = a.decay * rmean_c + (1.f - a.decay) * mean;
      if (a.rvar) a.rvar[c] = a.decay * rvar_c + (1.f - a.decay) * var * a.unbias;
    }
  }
  lds_barrier();
  const float mean = fin[0];
  const float g = gamma_c * inv_std(fin[1], a.eps);
  const float sh = fmaf(-mean, g, beta_c);

  // ---- normalize what the block holds
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  const uint32_t t2 = fresh(t);
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
    if (v < nvb) {
      const RawVec<T, VEC> r = slot(k);
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(r, j, g, sh);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mean), g, beta_c);
        }
      }
      store_vec<T, VEC>(y + chan_offset(a, c, sp, v, VEC), o);
    }
  }
}

namespace {

// Backward: (sum dy*xh, sum dy) of block sp of channel c from global memory,
// in that block's order (a thread's vectors ascending, elements ascending).
template <typename T, int VEC>
__device__ __forceinline__ void chan_pair_from_memory(const BnChanSplitArgs &a, uint32_t c,
                                                      uint32_t sp, float mean, float istd,
                                                      float nmi, float *red, float &sdx,
                                                      float &sdy) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  const uint32_t nvb = chan_block_samples(a, sp) * a.vpp.d;
  sdx = 0.f;
  sdy = 0.f;
#pragma unroll 1
  for (uint32_t v = threadIdx.x; v < nvb; v += kOnchipBlock) {
    const uint32_t off = chan_offset(a, c, sp, v, VEC);
    const RawVec<T, VEC> xr = load_raw<T, VEC>(x + off);
    const RawVec<T, VEC> dr = load_raw<T, VEC>(dy + off);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr, j, mean, istd, nmi);
      sdx = elem_fma<T, VEC>(dr, j, xh, sdx);
      sdy = elem_fma<T, VEC>(dr, j, a.one, sdy);
    }
  }
  chan_block_sum2(sdx, sdy, red);
}

} // namespace

// Backward (batch statistics).  With xh = (x-mean)*istd:
//   sdx = sum dy*xh (= dgamma), sdy = sum dy (= dbeta),
//   dx = dy*g*istd + xh*cA + cb,  cA = -istd*g*sdx/N + 2*dvar*std/N,
//   cb = -g*sdy*istd/N + dmean/N.
// NL vectors of x per thread: the first NL - NXS in registers, NXS in LDS; dy
// in batches of B, its first ND vectors per thread parked in LDS (NXS + ND <=
// 9: 144 KB), the others read again for dx.
template <typename T, int VEC, int NL, int NXS, int ND, int B>
__global__ void __launch_bounds__(kOnchipBlock)
bn_chan_split_bwd_kernel(const BnChanSplitArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  static_assert(NXS + ND <= 9 && NXS < NL, "LDS slots");
  constexpr int NXR = NL - NXS;
  __shared__ uint4 park[ND > 0 ? ND * kOnchipBlock : 1];
  __shared__ uint4 xlds[NXS > 0 ? NXS * kOnchipBlock : 1];
  __shared__ float red[32];
  __shared__ float got[2 * kChanSplitMax];
  __shared__ int miss[kChanSplitMax];
  __shared__ float fin[2];
  const uint32_t t = threadIdx.x;
  const uint32_t c = blockIdx.x / a.SP, sp = blockIdx.x % a.SP;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.dx);
  // (asked for ahead of the tensor)
  const float g = a.gamma ? a.gamma[c] : 1.f;
  const float mean = a.mean[c];
  const float vpe = a.var[c] + a.eps;
  const float p_dvar = a.dvar ? a.dvar[c] : 0.f;
  const float p_dmean = a.dmean ? a.dmean[c] : 0.f;
  const uint32_t nvb = chan_block_samples(a, sp) * a.vpp.d;
  const uint32_t last = nvb - 1u;

  RawVec<T, VEC> xr[NXR];
  {
    RawVec<T, VEC> xp[NXS > 0 ? NXS : 1];
#pragma unroll
    for (int k = 0; k < NXS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NXR + k) * kOnchipBlock + t;
      xp[k] = load_raw<T, VEC>(x + chan_offset(a, c, sp, min(v, last), VEC));
    }
#pragma unroll
    for (int k = 0; k < NXR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
      xr[k] = load_raw<T, VEC>(x + chan_offset(a, c, sp, min(v, last), VEC));
    }
#pragma unroll
    for (int k = 0; k < NXS; ++k) xlds[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, xp[k]);
  }
  // (each thread reads back only what it wrote: no barrier)
  auto xvec = [&](int k) -> RawVec<T, VEC> {
    if (k < NXR) return xr[k < NXR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, xlds[(k - NXR) * kOnchipBlock + t]);
  };
  const float istd = 1.0f / sqrtf(vpe);
  const float nmi = -mean * istd;

  // ---- pass 1: the block's (sum dy*xh, sum dy), vectors ascending
  float sdx = 0.f, sdy = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t t1 = fresh_after(t, sdx);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t1;
        d[i] = load_raw<T, VEC>(dy + chan_offset(a, c, sp, min(v, last), VEC));
      }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL) {
        if (k < ND) park[(k < ND ? k : 0) * kOnchipBlock + t] = __builtin_bit_cast(uint4, d[i]);
        if (static_cast<uint32_t>(k) * kOnchipBlock + t < nvb) {
          const RawVec<T, VEC> xk = xvec(k);
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float xh = norm_elem<T, VEC>(xk, j, mean, istd, nmi);
            sdx = elem_fma<T, VEC>(d[i], j, xh, sdx);
            sdy = elem_fma<T, VEC>(d[i], j, a.one, sdy);
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0); // the next batch's loads stay below: hoisted, the batches add up
  }
  chan_block_sum2(sdx, sdy, red);

  // ---- the partners' parts, the totals in block order, dgamma / dbeta
  chan_exchange(a, c, sp, sdx, sdy, got, miss);
  const uint64_t late = chan_missing(a, sp, miss);
  for (uint64_t todo = late; todo != 0; todo &= todo - 1) {
    const uint32_t p = static_cast<uint32_t>(__builtin_ctzll(todo));
    float px, py;
    chan_pair_from_memory<T, VEC>(a, c, p, mean, istd, nmi, red, px, py);
    if (t == 0) {
      got[2 * p] = px;
      got[2 * p + 1] = py;
    }
  }
  if (late != 0) lds_barrier();
  if (t == 0) {
    float tx = 0.f, ty = 0.f;
    for_pairs_in_order(got, 2, static_cast<int>(a.SP), [&](int, float px, float py) {
      tx += px;
      ty += py;
    });
    fin[0] = tx;
    fin[1] = ty;
    if (sp == 0) {
      if (a.dgamma) a.dgamma[c] = tx + (a.accum_g ? a.dgamma[c] : 0.f);
      if (a.dbeta) a.dbeta[c] = ty + (a.accum_b ? a.dbeta[c] : 0.f);
    }
  }
  if (dx == nullptr) return;
  lds_barrier();

  // ---- pass 2: dx = dy*gi + (x - mean)*A2 + cb  (half: x*A2 + B2, one mixed fma)
#pragma unroll
  for (int k = 0; k < NXR; ++k) forget<T, VEC>(xr[k]);
  const float cA = -istd * g * fin[0] * a.inv_N + (a.dvar ? 2.f * p_dvar * (vpe * istd) * a.inv_N : 0.f);
  const float cb = -g * fin[1] * istd * a.inv_N + (a.dmean ? p_dmean * a.inv_N : 0.f);
  const float gi = g * istd;
  const float A2 = istd * cA;
  const float B2 = sizeof(T) == 2 ? fmaf(nmi, cA, cb) : cb;
  auto emit = [&](const RawVec<T, VEC> &xv, const RawVec<T, VEC> &dv, uint32_t v) {
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
    T *dst = dx + chan_offset(a, c, sp, v, VEC);
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
    if (v < nvb) emit(xvec(k), __builtin_bit_cast(RawVec<T, VEC>, park[k * kOnchipBlock + t]), v);
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
        d[i] = load_raw<T, VEC>(dy + chan_offset(a, c, sp, min(v, last), VEC));
      }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t3;
      if (k < NL && v < nvb) {
        emit(xvec(k < NL ? k : 0), d[i], v);
        lastv = __builtin_bit_cast(float, __builtin_bit_cast(uint4, d[i]).x);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

namespace {

constexpr int kChanFwdMax = 25; // vectors per thread the forward holds (16 registers + 9 LDS)
constexpr int kChanBwdMax = 21; // vectors of x per thread the backward holds (12 registers + 9 LDS)

template <typename T, int VEC>
int run_chan_fwd(int nl, const BnChanSplitArgs &a, unsigned grid, hipStream_t st) {
#define CHAN_CASE(NR, NS)                                                                        \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH("bn_chan_split_fwd_kernel", (bn_chan_split_fwd_kernel<T, VEC, NR, NS>),       \
                   dim3(grid), dim3(kOnchipBlock), 0, st, a);                                    \
    return last_launch_status();                                                                 \
  }
  CHAN_CASE(2, 0)
  CHAN_CASE(4, 0)
  CHAN_CASE(7, 0)
  CHAN_CASE(10, 0)
  CHAN_CASE(13, 0)
  CHAN_CASE(16, 0)
  CHAN_CASE(16, 4)
  CHAN_CASE(16, 9)
#undef CHAN_CASE
  return NBLAHIP_EINVAL;
}

template <typename T, int VEC>
int run_chan_bwd(int nl, const BnChanSplitArgs &a, unsigned grid, hipStream_t st) {
  constexpr int kB = sizeof(T) == 2 ? 2 : 4;
#define CHAN_CASE(NL, NXS, ND)                                                                   \
  if (nl <= (NL)) {                                                                              \
    NBLAHIP_LAUNCH("bn_chan_split_bwd_kernel", (bn_chan_split_bwd_kernel<T, VEC, NL, NXS, ND, kB>), \
                   dim3(grid), dim3(kOnchipBlock), 0, st, a);                                    \
    return last_launch_status();                                                                 \
  }
  CHAN_CASE(2, 0, 2)
  CHAN_CASE(4, 0, 4)
  CHAN_CASE(7, 0, 7)
  CHAN_CASE(9, 0, 9)
  CHAN_CASE(12, 0, 9)
  CHAN_CASE(14, 2, 7)
  CHAN_CASE(16, 4, 5)
  CHAN_CASE(18, 6, 3)
  CHAN_CASE(21, 9, 0)
#undef CHAN_CASE
  return NBLAHIP_EINVAL;
}

// Shape test and the arguments both directions share; nl = vectors per thread.
bool chan_split_args(const BnProblem &p, bool backward, BnChanSplitArgs &a, int &nl) {
  if (!tune_int("BN_CHAN_SPLIT", 1)) return false;
  if (p.size2 <= 1 || p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.size2 % vec != 0 || !aligned16(p.x) || (p.out && !aligned16(p.out))) return false;
  if (backward && !aligned16(p.dy)) return false;
  if (p.size0 * p.C * p.size2 >= (int64_t{1} << 31)) return false;
  // A block whose partner's word does not arrive reads the partner's part of x
  // (and dy) again, which the partner may already be overwriting in place.
  const uint64_t tensor_bytes = static_cast<uint64_t>(p.size0 * p.C * p.size2) * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (ranges_overlap(p.out, p.x, tensor_bytes) || (backward && ranges_overlap(p.out, p.dy, tensor_bytes)))
    return false;
  // Short planes that share cache lines with the neighbouring channels' stay
  // with the kernels that put neighbouring channels on one XCD and store the
  // shared lines accordingly (bn_onchip.hip, the row kernels).
  const int64_t plane_bytes = p.size2 * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (plane_bytes % 128 != 0 && plane_bytes <= tune_int("BN_EDGE_STORES_MAX_BYTES", 1024)) return false;
  const int64_t cus = device_cus();
  const int64_t vpp = p.size2 / vec;
  const int64_t nv = p.size0 * vpp; // vectors of a channel
  // Channels the row kernels take whole (up to 8 vectors per thread of one
  // block) stay theirs: several to a block, no exchange.
  if (nv <= 8 * kOnchipBlock) return false;
  // The most blocks per channel that still fit the chip in one round; beyond
  // that (up to two rounds) only as far as the vectors per thread demand.
  const int max_nl = backward ? kChanBwdMax : kChanFwdMax;
  int64_t sp = 1;
  while (sp * 2 <= kChanSplitMax && p.C * sp * 2 <= cus && sp * 2 <= p.size0) sp *= 2;
  if (sp < 2) return false; // a channel per CU and more: bn_onchip.hip
  auto nl_of = [&](int64_t s) {
    const int64_t spb = (p.size0 + s - 1) / s;
    return (spb * vpp + kOnchipBlock - 1) / kOnchipBlock;
  };
  while (nl_of(sp) > max_nl && sp * 2 <= kChanSplitMax && p.C * sp * 2 <= 2 * cus && sp * 2 <= p.size0)
    sp *= 2;
  if (sp < 2 || nl_of(sp) > max_nl) return false;
  const int64_t spb = (p.size0 + sp - 1) / sp;
  if ((sp - 1) * spb >= p.size0) return false; // every block holds a sample
  // blocks for at least this share of the CUs: from the first channel on
  // ([32,C,56,56] half forward + backward, kernel time: 9.2 vs 25.9 us at C = 1,
  // 10.2 vs 26.8 at 12 against the split reduction's six launches)
  if (p.C * sp * 100 < cus * tune_int("BN_CHAN_SPLIT_MIN_PCT", 1)) return false;
  nl = static_cast<int>(nl_of(sp));
  a = BnChanSplitArgs{};
  a.x = p.x;
  a.gamma = p.gamma;
  a.C = static_cast<uint32_t>(p.C);
  a.size2 = static_cast<uint32_t>(p.size2);
  a.N = static_cast<uint32_t>(p.size0);
  a.SP = static_cast<uint32_t>(sp);
  a.spb = static_cast<uint32_t>(spb);
  a.vpp = FastDiv(static_cast<uint32_t>(vpp));
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  a.inv_N = static_cast<float>(1.0 / N);
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  a.spin = tune_int("XCHG_SPIN", 64) * 4;
  return true;
}

} // namespace

bool bn_chan_split_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnChanSplitArgs a;
  int nl = 0;
  if (!p.out || !chan_split_args(p, false, a, nl)) return false;
  a.y = p.out;
  a.beta = p.beta;
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  if (!xchg_acquire(static_cast<size_t>(a.C) * a.SP * 2, st, &a.xchg, &a.epoch, status)) return *status != 0;
  const unsigned grid = a.C * a.SP;
  *status = p.dtype == NBLAHIP_F16 ? run_chan_fwd<__half, 8>(nl, a, grid, st)
                                   : run_chan_fwd<float, 4>(nl, a, grid, st);
  return true;
}

bool bn_chan_split_bwd(const BnProblem &p, hipStream_t st, int *status) {
  BnChanSplitArgs a;
  int nl = 0;
  if (!p.batch_stat || (!p.out && !p.dgamma && !p.dbeta)) return false;
  if (!chan_split_args(p, true, a, nl)) return false;
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
  if (!xchg_acquire(static_cast<size_t>(a.C) * a.SP * 2, st, &a.xchg, &a.epoch, status)) return *status != 0;
  const unsigned grid = a.C * a.SP;
  *status = p.dtype == NBLAHIP_F16 ? run_chan_bwd<__half, 8>(nl, a, grid, st)
                                   : run_chan_bwd<float, 4>(nl, a, grid, st);
  return true;
}

} // namespace nblahip
