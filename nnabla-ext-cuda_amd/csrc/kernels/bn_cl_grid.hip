// Channel-last BatchNormalization training with the whole tensor held on the
// chip between the statistics and the normalization.
//
// x is [M][C].  A channel's column runs through every row, so no block can own
// a channel, and the split reduction reads x twice (statistics, then apply:
// 3 S forward, 5 S backward).  But the 256 CUs together hold 256 x 400 KB in
// registers and LDS - a [256,56,56,64] half tensor (103 MB) fits.  One
// 1024-thread block per CU takes a contiguous range of rows (NR 16-byte vectors
// per thread in registers, NS more in LDS, as in bn_onchip.hip); a thread's
// vectors always hold the same VEC channels (C / VEC divides 1024), so the
// per-channel sums are VEC accumulators per thread, folded over the block.
// The blocks then exchange their per-channel partials as {value, epoch} words
// (xchg.cuh) in two stages: block c merges the partials of channel c from all
// blocks (fixed order), writes mean / var / running statistics and publishes
// the result in eight copies (block b reads copy b % 8: all blocks polling the
// same C words queue up on the memory channel that holds them, a copy per block
// is 256 scattered stores per channel); every
// block reads its copy of the C results and normalizes what it holds: x
// crosses the memory system once (2 S).
//
// Every wait is a bounded poll.  A partial that does not turn up is computed
// by the block that needs it, from global memory, in the arithmetic of the
// block that owes it (same thread map, same order: the same bits); a channel
// result that does not turn up is merged by the block that needs it.  So every
// wave reaches the end whatever the other blocks do, and the results do not
// depend on who computed what.
#include <algorithm>
#include <type_traits>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"
#include "xchg.cuh"

namespace nblahip {

namespace {

constexpr int kGridMaxBlocks = 256; // partials per channel a block merges (one per thread of a wave quad)
constexpr int kGridMaxC = 128;      // channels (LDS fold of the per-channel sums) of the layouts that hold most
constexpr int kGridWideC = 512;     // channels of the layouts with three LDS slots fewer
// Copies of the per-channel results of stage 2; block b reads copy b % 8.  A
// copy per block (256 scattered 8-byte stores per channel) made the second hop
// three times as slow as the first, one copy for all makes every block poll the
// same eight cache lines ([256,56,56,64] half forward / backward: 49.1 / 76.0 us
// with 256 copies, 46.9 / 75.0 with 8, 48.4 / 76.0 with one).
constexpr uint32_t kGridCopies = 8;

struct BnClGridArgs {
  const void *x;
  void *y;
  const float *gamma, *beta;
  float *mean, *var, *rmean, *rvar;
  uint32_t C;
  uint32_t cv;      // channel vectors per row = C / VEC (a power of two)
  uint32_t nv;      // vectors of the tensor = M * cv
  uint32_t vb;      // vectors per block (whole rows)
  uint32_t nblocks;
  float inv_N, unbias, decay, eps, one;
  // backward
  const void *dy;
  void *dx;                  // may be null
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;     // may be null
  int accum_dx, accum_g, accum_b;
  unsigned long long *x1; // stage 1: [nblocks][C][2] = (mean, m2) of the block's rows
                          //          (backward: (sum dy*xh, sum dy))
  unsigned long long *x2; // stage 2: [copies][C][2] = (mean, var)
  uint32_t epoch;
  int spin;
  uint32_t copies; // copies of the stage-2 results; block b reads copy b % copies
};

// Vectors of block b.
__device__ __forceinline__ uint32_t grid_block_vectors(const BnClGridArgs &a, uint32_t b) {
  const uint32_t first = b * a.vb;
  return first >= a.nv ? 0u : min(a.vb, a.nv - first);
}

// Per-channel totals of v[VEC] over the threads of the block that hold the
// same channel vector (t % cv): butterfly over the lanes cv apart, one row of
// fold[16][C] per wave, the rows added in wave order by one thread per channel
// (tot[C]), and every thread reads back its channels' totals.
// (No barrier ahead of the first write: every earlier reader of fold has passed
// the last barrier of the call before, and so has every reader of tot by the
// time tot is written again, two barriers further on.)
template <int VEC>
__device__ __forceinline__ void grid_channel_sums(float (&v)[VEC], uint32_t cv, uint32_t cvx,
                                                  float *fold, float *tot, uint32_t C) {
  constexpr int NW = kOnchipBlock / kWave;
  lanes_sum_from<VEC>(v, cv); // (a step at a time for all values, off the LDS crossbar: xor_add)
  if ((threadIdx.x & (kWave - 1)) < cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fold[(threadIdx.x / kWave) * C + cvx * VEC + j] = v[j];
  }
  lds_barrier();
  if (threadIdx.x < C) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w * C + threadIdx.x];
    tot[threadIdx.x] = t;
  }
  lds_barrier();
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = tot[cvx * VEC + j];
}

// The same fold for ONE channel (element e of the vectors of channel vector
// c / VEC): identical butterfly and wave order, so identical bits.
__device__ __forceinline__ float grid_channel_sum1(float v, uint32_t cv, uint32_t cvx, uint32_t c,
                                                   bool mine, float *fold, uint32_t C) {
  constexpr int NW = kOnchipBlock / kWave;
  v = lanes_sum_from(v, cv);
  lds_barrier(); // earlier readers of fold are done
  if ((threadIdx.x & (kWave - 1)) < cv && mine) fold[(threadIdx.x / kWave) * C + c] = v;
  lds_barrier();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) t += fold[w * C + c];
  return t;
}

// (mean, m2) of the rows of block p for channel c, from global memory, in the
// order block p itself uses (its thread map, slots ascending per thread, the
// thread's own mean as the shift, the same folds): what block p publishes for
// c, bit for bit.  Only the threads of c's channel vector load (the folds
// never mix channel vectors) and only c's element is accumulated, so this
// costs a handful of registers.
template <typename T, int VEC>
__device__ __forceinline__ void grid_partial_from_memory(const BnClGridArgs &a, uint32_t p,
                                                         uint32_t c, float *fold, float &m,
                                                         float &q) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const uint32_t t = threadIdx.x;
  const uint32_t cvx = t % a.cv, e = c % VEC;
  const uint32_t vbb = grid_block_vectors(a, p);
  const bool mine = cvx == c / VEC;
  const uint32_t vbp = mine ? vbb : 0u;
  const size_t first = static_cast<size_t>(p) * a.vb;
  float s = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll 1
  for (uint32_t v = t; v < vbp; v += kOnchipBlock) {
    const RawVec<T, VEC> r = load_raw<T, VEC>(x + (first + v) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float n = elem_fma<T, VEC>(r, j, a.one, s);
      s = static_cast<uint32_t>(j) == e ? n : s;
    }
  }
  const float nt = (mine && t < vbb) ? static_cast<float>((vbb - 1u - t) / kOnchipBlock + 1u) : 0.f;
  const float kk = s * (1.0f / fmaxf(nt, 1.f));
#pragma unroll 1
  for (uint32_t v = t; v < vbp; v += kOnchipBlock) {
    const RawVec<T, VEC> r = load_raw<T, VEC>(x + (first + v) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = elem_fma<T, VEC>(r, j, a.one, -kk);
      const float n1 = s1 + d;
      const float n2 = fmaf(d, d, s2);
      s1 = static_cast<uint32_t>(j) == e ? n1 : s1;
      s2 = static_cast<uint32_t>(j) == e ? n2 : s2;
    }
  }
  m = grid_channel_sum1(s, a.cv, cvx, c, mine, fold, a.C);
  m *= 1.0f / static_cast<float>(vbb / a.cv);
  const float d = kk - m;
  q = grid_channel_sum1(mine ? fmaf(d, fmaf(nt, d, 2.f * s1), s2) : 0.f, a.cv, cvx, c, mine, fold, a.C);
}

// Merged (mean, var) of channel c over all blocks: thread p < nblocks takes
// block p's partial (polled; computed here if it does not arrive), the block
// merges them in a fixed order.  Same result in every thread and in every block
// that calls it.  scratch: miss[kGridMaxBlocks] ints, got[2 * kGridMaxBlocks],
// wel[3 * 16], fold[16 * C].
template <typename T, int VEC>
__device__ __forceinline__ void grid_channel_result(const BnClGridArgs &a, uint32_t c, int *miss,
                                                    float *got, float *wel, float *fold,
                                                    float &mean, float &var) {
  const uint32_t t = threadIdx.x;
  lds_barrier(); // got / miss of an earlier call have been consumed
  if (t == 0) miss[kGridMaxBlocks] = 0; // any partial missing at all?
  lds_barrier();
  if (t < a.nblocks) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x1 + (static_cast<size_t>(t) * a.C + c) * 2, a.epoch, a.spin, &v0, &v1);
    got[2 * t] = v0;
    got[2 * t + 1] = v1;
    miss[t] = ok ? 0 : 1;
    if (!ok) miss[kGridMaxBlocks] = 1;
  }
  lds_barrier();
  for (uint32_t p = 0; miss[kGridMaxBlocks] && p < a.nblocks; ++p) {
    if (!miss[p]) continue; // same answer in every thread
    float m, q;
    grid_partial_from_memory<T, VEC>(a, p, c, fold, m, q);
    if (t == 0) {
      got[2 * p] = m;
      got[2 * p + 1] = q;
    }
    lds_barrier();
  }
  // mean = sum n_p * mean_p / N, m2 = sum (m2_p + n_p * (mean_p - mean)^2): two
  // block sums in a fixed order (a Chan merge tree over 256 partials took 2.5 us)
  float np = 0.f, mp = 0.f, qp = 0.f;
  if (t < a.nblocks) {
    mp = got[2 * t];
    qp = got[2 * t + 1];
    np = static_cast<float>(grid_block_vectors(a, t) / a.cv);
  }
  mean = onchip_block_sum(np * mp, wel) * a.inv_N;
  const float d = mp - mean;
  var = onchip_block_sum(fmaf(np * d, d, qp), wel) * a.inv_N;
}

// Backward: (sum dy*xh, sum dy) of the rows of block p for channel c, from
// global memory, in block p's own order (vectors k * 1024 + t ascending per
// thread, the same folds): what block p publishes for c, bit for bit.
template <typename T, int VEC>
__device__ __forceinline__ void grid_pair_from_memory(const BnClGridArgs &a, uint32_t p,
                                                      uint32_t c, float *fold, float &sdx,
                                                      float &sdy) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  const uint32_t t = threadIdx.x;
  const uint32_t cvx = t % a.cv, e = c % VEC;
  const uint32_t vbp = cvx == c / VEC ? grid_block_vectors(a, p) : 0u;
  const size_t first = static_cast<size_t>(p) * a.vb;
  const float mean = a.mean[c];
  const float istd = 1.0f / sqrtf(a.var[c] + a.eps);
  const float nmi = -mean * istd;
  sdx = 0.f;
  sdy = 0.f;
#pragma unroll 1
  for (uint32_t v = t; v < vbp; v += kOnchipBlock) {
    const RawVec<T, VEC> xr = load_raw<T, VEC>(x + (first + v) * VEC);
    const RawVec<T, VEC> dr = load_raw<T, VEC>(dy + (first + v) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr, j, mean, istd, nmi);
      const float nx = elem_fma<T, VEC>(dr, j, xh, sdx);
      const float ny = elem_fma<T, VEC>(dr, j, a.one, sdy);
      sdx = static_cast<uint32_t>(j) == e ? nx : sdx;
      sdy = static_cast<uint32_t>(j) == e ? ny : sdy;
    }
  }
  sdx = grid_channel_sum1(sdx, a.cv, cvx, c, cvx == c / VEC, fold, a.C);
  sdy = grid_channel_sum1(sdy, a.cv, cvx, c, cvx == c / VEC, fold, a.C);
}

// Backward: (sum dy*xh, sum dy) of channel c over all blocks, in block order.
// Same structure and scratch as grid_channel_result.
template <typename T, int VEC>
__device__ __forceinline__ void grid_pair_result(const BnClGridArgs &a, uint32_t c, int *miss,
                                                 float *got, float *wel, float *fold, float &sdx,
                                                 float &sdy) {
  const uint32_t t = threadIdx.x;
  lds_barrier(); // got / miss of an earlier call have been consumed
  if (t == 0) miss[kGridMaxBlocks] = 0;
  lds_barrier();
  if (t < a.nblocks) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x1 + (static_cast<size_t>(t) * a.C + c) * 2, a.epoch, a.spin, &v0, &v1);
    got[2 * t] = v0;
    got[2 * t + 1] = v1;
    miss[t] = ok ? 0 : 1;
    if (!ok) miss[kGridMaxBlocks] = 1;
  }
  lds_barrier();
  for (uint32_t p = 0; miss[kGridMaxBlocks] && p < a.nblocks; ++p) {
    if (!miss[p]) continue; // same answer in every thread
    float px, py;
    grid_pair_from_memory<T, VEC>(a, p, c, fold, px, py);
    if (t == 0) {
      got[2 * p] = px;
      got[2 * p + 1] = py;
    }
    lds_barrier();
  }
  sdx = onchip_block_sum(t < a.nblocks ? got[2 * t] : 0.f, wel);
  sdy = onchip_block_sum(t < a.nblocks ? got[2 * t + 1] : 0.f, wel);
}

} // namespace

template <typename T, int VEC, int NR, int NS, int CMAX>
__global__ void __launch_bounds__(kOnchipBlock)
bn_cl_grid_fwd_kernel(const BnClGridArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float fold[16 * CMAX];
  __shared__ float tot[CMAX];
  __shared__ float fin[2 * CMAX];   // (mean, var) per channel
  __shared__ float got[2 * kGridMaxBlocks];
  __shared__ int miss[kGridMaxBlocks + 2]; // [kGridMaxBlocks], [+1]: any partial / any result missing
  __shared__ float wel[3 * 16];
  __shared__ float gb[2 * CMAX]; // gamma, beta
  const uint32_t b = blockIdx.x;
  const uint32_t t = threadIdx.x;
  // gamma and beta of channel t, asked for ahead of the tensor (behind the
  // exchange they would cost a memory round trip of their own)
  float gamma_t = 1.f, beta_t = 0.f;
  if (t < a.C) {
    if (a.gamma) gamma_t = a.gamma[t];
    if (a.beta) beta_t = a.beta[t];
  }
  const uint32_t cvx = t % a.cv;
  const uint32_t ch = cvx * VEC;
  const uint32_t vbb = grid_block_vectors(a, b);
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(b) * a.vb * VEC;
  T *__restrict__ y = static_cast<T *>(a.y) + static_cast<size_t>(b) * a.vb * VEC;

  // ---- loads: slot k is vector k * 1024 + t of the block (a slot past the
  // block's end reads the block's last vector and stays out of sums and stores)
  const uint32_t last = vbb - 1;
  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t;
      parked[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
      raw[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
    if (t < a.C) { // (they arrive first; read behind the barriers of the folds)
      gb[t] = gamma_t;
      gb[CMAX + t] = beta_t;
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };

  // (slot k holds a vector of the block: t against a scalar, no register per slot)
  auto holds = [&](int k) { return static_cast<int>(t) < static_cast<int>(vbb) - k * kOnchipBlock; };

  // ---- this block's partial per channel, from sums every wave takes over its
  // OWN registers as its loads arrive (the memory system serves a CU's waves
  // one after the other, 2 to 18 us after the start here: what a wave does
  // before the block's first barrier hides behind the other waves' loads, what
  // comes after it keeps memory idle - a second pass about the block's mean
  // cost 5.8 us of [256,56,56,64]'s 49).  Per thread and channel: s = sum x,
  // then about the thread's own mean K = s / n: s1 = sum (x - K) (rounding
  // residue), s2 = sum (x - K)^2.  Then mean = sum_t s / rows, and about it
  // m2 = sum_t (s2 + 2 e s1 + n e^2), e = K - mean: two block sums of a few
  // operations per thread.  sum_t n e^2 is the variance between the threads'
  // means, never more than m2 itself: nothing cancels, whatever the data.
  float m[VEC], q[VEC];
  {
    float kk[VEC], s1[VEC], s2[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) m[j] = s1[j] = s2[j] = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (holds(k)) {
        const RawVec<T, VEC> r = slot(k);
#pragma unroll
        for (int j = 0; j < VEC; ++j) m[j] = elem_fma<T, VEC>(r, j, a.one, m[j]);
      }
    }
    const float nt = t < vbb ? static_cast<float>((vbb - 1u - t) / kOnchipBlock + 1u) : 0.f;
    const float rnt = 1.0f / fmaxf(nt, 1.f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) kk[j] = m[j] * rnt;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (holds(k)) {
        const RawVec<T, VEC> r = slot(k);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(r, j, a.one, -kk[j]);
          s1[j] += d;
          s2[j] = fmaf(d, d, s2[j]);
        }
      }
    }
    grid_channel_sums<VEC>(m, a.cv, cvx, fold, tot, a.C);
    const float icnt = 1.0f / static_cast<float>(vbb / a.cv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      m[j] *= icnt;
      const float e = kk[j] - m[j];
      q[j] = fmaf(e, fmaf(nt, e, 2.f * s1[j]), s2[j]);
    }
    grid_channel_sums<VEC>(q, a.cv, cvx, fold, tot, a.C);
  }
  // publish (mean, m2) of every channel: a word per thread (through fin, which
  // is free until the results arrive)
  if (t < a.cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      fin[2 * (ch + j)] = m[j];
      fin[2 * (ch + j) + 1] = q[j];
    }
  }
  lds_barrier();
  for (uint32_t e = t; e < 2 * a.C; e += kOnchipBlock)
    xchg_publish(a.x1 + static_cast<size_t>(b) * a.C * 2 + e, fin[e], a.epoch);

  // ---- stage 2: block c merges channel c, writes its statistics, publishes
  for (uint32_t c = b; c < a.C; c += a.nblocks) {
    float mean, var;
    grid_channel_result<T, VEC>(a, c, miss, got, wel, fold, mean, var);
    if (t == 0) {
      a.mean[c] = mean;
      a.var[c] = var;
      if (a.rmean) a.rmean[c] = a.decay * a.rmean[c] + (1.f - a.decay) * mean;
      if (a.rvar) a.rvar[c] = a.decay * a.rvar[c] + (1.f - a.decay) * var * a.unbias;
    }
    if (t < a.copies) { // copy t
      unsigned long long *w = a.x2 + (static_cast<size_t>(t) * a.C + c) * 2;
      xchg_publish(w, mean, a.epoch);
      xchg_publish(w + 1, var, a.epoch);
    }
  }

  // ---- every block: the C results (merged here where one does not arrive)
  lds_barrier();
  if (t == 0) miss[kGridMaxBlocks + 1] = 0;
  lds_barrier();
  for (uint32_t c = t; c < a.C; c += kOnchipBlock) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x2 + (static_cast<size_t>(b % a.copies) * a.C + c) * 2, a.epoch, a.spin, &v0, &v1);
    fin[2 * c] = v0;
    fin[2 * c + 1] = ok ? v1 : -1.f; // a variance is never negative: marks "missing"
    if (!ok) miss[kGridMaxBlocks + 1] = 1;
  }
  lds_barrier();
  for (uint32_t c = 0; miss[kGridMaxBlocks + 1] && c < a.C; ++c) {
    if (fin[2 * c + 1] >= 0.f) continue; // same answer in every thread
    float mean, var;
    grid_channel_result<T, VEC>(a, c, miss, got, wel, fold, mean, var);
    lds_barrier();
    if (t == 0) {
      fin[2 * c] = mean;
      fin[2 * c + 1] = var;
    }
    lds_barrier();
  }

  // ---- normalize what the block holds
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  float sc[VEC], sh[VEC], mu[VEC], be[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mu[j] = fin[2 * (ch + j)];
    sc[j] = gb[ch + j] * inv_std(fin[2 * (ch + j) + 1], a.eps);
    be[j] = gb[CMAX + ch + j];
    sh[j] = fmaf(-mu[j], sc[j], be[j]);
  }
  const uint32_t t2 = fresh(t);
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
    if (v < vbb) {
      const RawVec<T, VEC> r = slot(k);
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(r, j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mu[j]), sc[j], be[j]);
        }
      }
      store_vec<T, VEC>(y + static_cast<size_t>(v) * VEC, o);
    }
  }
}

// Backward (batch statistics).  With xh = (x-mean)*istd per channel:
//   sdx = sum dy*xh (= dgamma), sdy = sum dy (= dbeta),
//   dx = dy*g*istd + xh*cA + cb,  cA = -istd*g*sdx/N + 2*dvar*std/N,
//   cb = -g*sdy*istd/N + dmean/N.
// x is held as in the forward (NR + NS vectors per thread; what a block has
// beyond that is streamed with dy in both passes), dy is streamed twice in
// batches of B vectors; the blocks exchange (sdx, sdy) per channel in the
// forward's two stages, block c writing dgamma[c] / dbeta[c].
template <typename T, int VEC, int NR, int NS, int B, int CMAX>
__global__ void __launch_bounds__(kOnchipBlock)
bn_cl_grid_bwd_kernel(const BnClGridArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float fold[16 * CMAX];
  __shared__ float tot[CMAX];
  __shared__ float fin[2 * CMAX]; // (sdx, sdy) totals per channel
  __shared__ int finmiss[CMAX];
  __shared__ float got[2 * kGridMaxBlocks];
  __shared__ int miss[kGridMaxBlocks + 2];
  __shared__ float wel[16];
  __shared__ float par[5 * CMAX]; // mean, var, gamma, dvar, dmean
  const uint32_t b = blockIdx.x;
  const uint32_t t = threadIdx.x;
  // The parameters of channel t, asked for ahead of the tensor: behind the LDS
  // stores of x, or behind the exchange, each would cost a memory round trip
  // of its own.
  float p_mean = 0.f, p_var = 1.f, p_gamma = 1.f, p_dvar = 0.f, p_dmean = 0.f;
  if (t < a.C) {
    p_mean = a.mean[t];
    p_var = a.var[t];
    if (a.gamma) p_gamma = a.gamma[t];
    if (a.dvar) p_dvar = a.dvar[t];
    if (a.dmean) p_dmean = a.dmean[t];
  }
  const uint32_t cvx = t % a.cv;
  const uint32_t ch = cvx * VEC;
  const uint32_t vbb = grid_block_vectors(a, b);
  const size_t base = static_cast<size_t>(b) * a.vb * VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + base;
  T *__restrict__ dx = a.dx ? static_cast<T *>(a.dx) + base : nullptr;
  const uint32_t last = vbb - 1;

  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t;
      parked[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
      raw[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };
  if (t < a.C) {
    par[t] = p_mean;
    par[CMAX + t] = p_var;
    par[2 * CMAX + t] = p_gamma;
    par[3 * CMAX + t] = p_dvar;
    par[4 * CMAX + t] = p_dmean;
  }
  lds_barrier();
  float mean[VEC], istd[VEC], nmi[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mean[j] = par[ch + j];
    istd[j] = 1.0f / sqrtf(par[CMAX + ch + j] + a.eps);
    nmi[j] = -mean[j] * istd[j];
  }

  // ---- pass 1: the block's (sum dy*xh, sum dy) per channel, vectors ascending
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t t1 = fresh_after(t, sdx[0]);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const uint32_t v = static_cast<uint32_t>(k0 + i) * kOnchipBlock + t1;
      d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL && static_cast<uint32_t>(k) * kOnchipBlock + t < vbb) {
        const RawVec<T, VEC> xr = slot(k);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr, j, mean[j], istd[j], nmi[j]);
          sdx[j] = elem_fma<T, VEC>(d[i], j, xh, sdx[j]);
          sdy[j] = elem_fma<T, VEC>(d[i], j, a.one, sdy[j]);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0); // the next batch's loads stay below: hoisted, the batches add up
  }
#pragma unroll 1
  for (uint32_t v = static_cast<uint32_t>(NL) * kOnchipBlock + t; v < vbb; v += kOnchipBlock) {
    const RawVec<T, VEC> xr = load_raw<T, VEC>(x + static_cast<size_t>(v) * VEC);
    const RawVec<T, VEC> dr = load_raw<T, VEC>(dy + static_cast<size_t>(v) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr, j, mean[j], istd[j], nmi[j]);
      sdx[j] = elem_fma<T, VEC>(dr, j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dr, j, a.one, sdy[j]);
    }
  }
  grid_channel_sums<VEC>(sdx, a.cv, cvx, fold, tot, a.C);
  if (t < a.cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fin[ch + j] = sdx[j];
  }
  grid_channel_sums<VEC>(sdy, a.cv, cvx, fold, tot, a.C);
  // (fin's stores precede the barriers of the second fold: visible by now)
  for (uint32_t e = t; e < 2 * a.C; e += kOnchipBlock)
    xchg_publish(a.x1 + static_cast<size_t>(b) * a.C * 2 + e, (e & 1) ? tot[e >> 1] : fin[e >> 1], a.epoch);

  // ---- stage 2: block c sums channel c over the blocks, writes dgamma / dbeta, publishes
  for (uint32_t c = b; c < a.C; c += a.nblocks) {
    float tx, ty;
    grid_pair_result<T, VEC>(a, c, miss, got, wel, fold, tx, ty);
    if (t == 0) {
      if (a.dgamma) a.dgamma[c] = tx + (a.accum_g ? a.dgamma[c] : 0.f);
      if (a.dbeta) a.dbeta[c] = ty + (a.accum_b ? a.dbeta[c] : 0.f);
    }
    if (t < a.copies) { // copy t
      unsigned long long *w = a.x2 + (static_cast<size_t>(t) * a.C + c) * 2;
      xchg_publish(w, tx, a.epoch);
      xchg_publish(w + 1, ty, a.epoch);
    }
  }
  if (dx == nullptr) return;

  // ---- every block: the C totals (summed here where one does not arrive)
  lds_barrier();
  if (t == 0) miss[kGridMaxBlocks + 1] = 0;
  lds_barrier();
  for (uint32_t c = t; c < a.C; c += kOnchipBlock) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x2 + (static_cast<size_t>(b % a.copies) * a.C + c) * 2, a.epoch, a.spin, &v0, &v1);
    fin[2 * c] = v0;
    fin[2 * c + 1] = v1;
    finmiss[c] = ok ? 0 : 1;
    if (!ok) miss[kGridMaxBlocks + 1] = 1;
  }
  lds_barrier();
  for (uint32_t c = 0; miss[kGridMaxBlocks + 1] && c < a.C; ++c) {
    if (!finmiss[c]) continue; // same answer in every thread
    float tx, ty;
    grid_pair_result<T, VEC>(a, c, miss, got, wel, fold, tx, ty);
    lds_barrier();
    if (t == 0) {
      fin[2 * c] = tx;
      fin[2 * c + 1] = ty;
    }
    lds_barrier();
  }

  // ---- pass 2: dx = dy*gi + (x - mean)*A2 + cb  (half: x*A2 + B2, one mixed fma)
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  float gi[VEC], A2[VEC], B2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const float g = par[2 * CMAX + ch + j];
    const float vpe = par[CMAX + ch + j] + a.eps;
    const float cA = -istd[j] * g * fin[2 * (ch + j)] * a.inv_N +
                     (a.dvar ? 2.f * par[3 * CMAX + ch + j] * (vpe * istd[j]) * a.inv_N : 0.f);
    const float cb = -g * fin[2 * (ch + j) + 1] * istd[j] * a.inv_N +
                     (a.dmean ? par[4 * CMAX + ch + j] * a.inv_N : 0.f);
    gi[j] = g * istd[j];
    A2[j] = istd[j] * cA;
    B2[j] = sizeof(T) == 2 ? fmaf(nmi[j], cA, cb) : cb;
  }
  auto emit = [&](const RawVec<T, VEC> &xr, const RawVec<T, VEC> &dr, uint32_t v) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float xt;
      if constexpr (sizeof(T) == 2) {
        xt = elem_fma<T, VEC>(xr, j, A2[j], B2[j]);
      } else {
        xt = fmaf(elem_fma<T, VEC>(xr, j, a.one, -mean[j]), A2[j], B2[j]);
      }
      o[j] = elem_fma<T, VEC>(dr, j, gi[j], xt);
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
  float lastv = B2[0];
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t t2 = fresh_after(t, lastv);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const uint32_t v = static_cast<uint32_t>(k0 + i) * kOnchipBlock + t2;
      d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(v, last)) * VEC);
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
      if (k < NL && v < vbb) {
        emit(slot(k), d[i], v);
        lastv = __builtin_bit_cast(float, __builtin_bit_cast(uint4, d[i]).x);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll 1
  for (uint32_t v = static_cast<uint32_t>(NL) * kOnchipBlock + t; v < vbb; v += kOnchipBlock) {
    const RawVec<T, VEC> xr = load_raw<T, VEC>(x + static_cast<size_t>(v) * VEC);
    const RawVec<T, VEC> dr = load_raw<T, VEC>(dy + static_cast<size_t>(v) * VEC);
    emit(xr, dr, v);
  }
}

namespace {

template <typename T, int VEC>
int run_grid_fwd(int nl, const BnClGridArgs &a, hipStream_t st) {
#define GRID_CASE(NR, NS, CMAX)                                                                  \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH("bn_cl_grid_fwd_kernel", (bn_cl_grid_fwd_kernel<T, VEC, NR, NS, CMAX>),       \
                   dim3(a.nblocks), dim3(kOnchipBlock), 0, st, a);                               \
    return last_launch_status();                                                                 \
  }
  if (a.C <= static_cast<uint32_t>(kGridMaxC)) {
    GRID_CASE(4, 0, kGridMaxC)
    GRID_CASE(8, 0, kGridMaxC)
    GRID_CASE(12, 0, kGridMaxC)
    GRID_CASE(16, 0, kGridMaxC)
    GRID_CASE(16, 3, kGridMaxC)
    GRID_CASE(16, 6, kGridMaxC)
    GRID_CASE(16, 9, kGridMaxC)
  } else { // the per-channel arrays take 32 KB more of LDS
    GRID_CASE(4, 0, kGridWideC)
    GRID_CASE(8, 0, kGridWideC)
    GRID_CASE(12, 0, kGridWideC)
    GRID_CASE(16, 0, kGridWideC)
    GRID_CASE(16, 3, kGridWideC)
    GRID_CASE(16, 6, kGridWideC)
  }
#undef GRID_CASE
  return NBLAHIP_EINVAL;
}

} // namespace

namespace {

template <typename T, int VEC>
int run_grid_bwd(int nl, const BnClGridArgs &a, hipStream_t st) {
  constexpr int B = sizeof(T) == 2 ? 2 : 4;
#define GRID_CASE(NR, NS, CMAX)                                                                  \
  if (nl <= (NR) + (NS)) {                                                                       \
    constexpr int kNS = (NS) > 9 ? ((CMAX) > kGridMaxC ? 6 : 9) : (NS);                          \
    NBLAHIP_LAUNCH("bn_cl_grid_bwd_kernel", (bn_cl_grid_bwd_kernel<T, VEC, NR, kNS, B, CMAX>),   \
                   dim3(a.nblocks), dim3(kOnchipBlock), 0, st, a);                               \
    return last_launch_status();                                                                 \
  }
  if (a.C <= static_cast<uint32_t>(kGridMaxC)) {
    GRID_CASE(4, 0, kGridMaxC)
    GRID_CASE(8, 0, kGridMaxC)
    GRID_CASE(12, 0, kGridMaxC)
    GRID_CASE(12, 3, kGridMaxC)
    GRID_CASE(12, 6, kGridMaxC)
    // (more per thread than the 21 vectors held: the rest is streamed with dy)
    GRID_CASE(12, 1 << 20, kGridMaxC)
  } else {
    GRID_CASE(4, 0, kGridWideC)
    GRID_CASE(8, 0, kGridWideC)
    GRID_CASE(12, 0, kGridWideC)
    GRID_CASE(12, 3, kGridWideC)
    GRID_CASE(12, 1 << 20, kGridWideC)
  }
#undef GRID_CASE
  return NBLAHIP_EINVAL;
}

// Shape test and the arguments both directions share; nl = vectors per thread.
bool grid_args(const BnProblem &p, BnClGridArgs &a, int &nl) {
  if (!tune_int("BN_CL_GRID", 1)) return false;
  if (p.size2 != 1 || p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.C % vec != 0 || p.C > kGridWideC || !aligned16(p.x) || (p.out && !aligned16(p.out))) return false;
  // 129 - 512 channels: from the rows on that the split kernels' backward no
  // longer holds (36 blocks of 1024 rows); below, those take both directions
  // ([128,14,14,512] half 17.8 / 20.0 us against 23.6 / 30.5 us here).
  if (p.C > kGridMaxC &&
      (!tune_int("BN_CL_GRID_WIDE", 1) || p.size0 < tune_int("BN_CL_GRID_WIDE_MIN_ROWS", 36865)))
    return false;
  const int64_t cv = p.C / vec;
  if ((cv & (cv - 1)) != 0 || cv > kWave) return false;
  // A block whose partner's word does not arrive reads the partner's rows of x
  // (and dy) again, which the partner may already be overwriting in place.
  const uint64_t tensor_bytes = static_cast<uint64_t>(p.size0 * p.C) * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (ranges_overlap(p.out, p.x, tensor_bytes) || ranges_overlap(p.out, p.dy, tensor_bytes)) return false;
  const int64_t M = p.size0;
  const int blocks = std::min(device_cus(), kGridMaxBlocks);
  // whole rows per block, the same for every block but the last
  const int64_t rows_pb = (M + blocks - 1) / blocks;
  const int64_t vb = rows_pb * cv;
  nl = static_cast<int>((vb + kOnchipBlock - 1) / kOnchipBlock);
  const int64_t nblocks = (M + rows_pb - 1) / rows_pb;
  // Up to what the chip holds, and from 8192 rows: below, the split kernels
  // (a block per 1024 rows) are as fast or faster.  Kernel time of forward +
  // backward, this against the split kernels / the split reduction, half
  // [M, 64]: 22.8 vs 21.9 us at M = 6272, 23.1 vs 29.1 at 12544, 24.8 vs 32.9 at
  // 50176, 29.5 vs 45.5 at 100352, 33.6 vs 55.0 at 150528; float 19.5 vs 18.6,
  // 20.0 vs 22.2, 24.2 vs 31.5; [M, 128] half 24.1 vs 22.5 at 6272, 25.1 vs 29.4
  // at 12544.
  if (nl < tune_int("BN_CL_GRID_MIN_SLOTS", 1) || nl > 25 || nblocks < blocks / 2) return false;
  if (M < tune_int("BN_CL_GRID_MIN_ROWS", 8192)) return false;
  a = BnClGridArgs{};
  a.x = p.x;
  a.gamma = p.gamma;
  a.C = static_cast<uint32_t>(p.C);
  a.cv = static_cast<uint32_t>(cv);
  a.nv = static_cast<uint32_t>(M * cv);
  a.vb = static_cast<uint32_t>(vb);
  a.nblocks = static_cast<uint32_t>(nblocks);
  const double N = static_cast<double>(M);
  a.inv_N = static_cast<float>(1.0 / N);
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  a.spin = tune_int("XCHG_SPIN", 64) * 16; // a whole-chip exchange: wait longer before recomputing
  a.copies = std::min<uint32_t>(kGridCopies, a.nblocks);
  return true;
}

// Exchange words of both stages.
bool grid_exchange(const BnProblem &p, BnClGridArgs &a, hipStream_t st, int *status) {
  const size_t words = static_cast<size_t>(a.nblocks + a.copies) * p.C * 2;
  if (!xchg_acquire(words, st, &a.x1, &a.epoch, status)) return false;
  a.x2 = a.x1 + static_cast<size_t>(a.nblocks) * p.C * 2;
  return true;
}

} // namespace

bool bn_cl_grid_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnClGridArgs a;
  int nl = 0;
  if (!p.out || !grid_args(p, a, nl)) return false;
  if (p.C > kGridMaxC && nl > 22) return false; // (the wide layouts hold 16 + 6 vectors)
  a.y = p.out;
  a.beta = p.beta;
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  if (!grid_exchange(p, a, st, status)) return *status != 0;
  *status = p.dtype == NBLAHIP_F16 ? run_grid_fwd<__half, 8>(nl, a, st) : run_grid_fwd<float, 4>(nl, a, st);
  return true;
}

bool bn_cl_grid_bwd(const BnProblem &p, hipStream_t st, int *status) {
  BnClGridArgs a;
  int nl = 0;
  if (!p.batch_stat || !tune_int("BN_CL_GRID_BWD", 1) || !grid_args(p, a, nl)) return false;
  if (!aligned16(p.dy)) return false;
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
  if (!grid_exchange(p, a, st, status)) return *status != 0;
  *status = p.dtype == NBLAHIP_F16 ? run_grid_bwd<__half, 8>(nl, a, st) : run_grid_bwd<float, 4>(nl, a, st);
  return true;
}

} // namespace nblahip
