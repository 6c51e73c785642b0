// Channel-last BatchNormalization training with the whole tensor held on the
// chip between the statistics and the normalization.
//
// x is [M][C].  A channel's column runs through every row, so no block can own
// a channel, and the split reduction reads x twice (statistics, then apply:
// 3 S forward, 5 S backward).  But the 256 CUs together hold 256 x 400 KB in
// registers and LDS - a [256,56,56,64] half tensor (103 MB) fits.  One
// 1024-thread block per CU takes a range of rows of one column strip (a strip
// is a power of two of 16-byte vectors wide, at most 128 channels; a tensor of
// up to 128 channels is one strip and the block's rows are contiguous memory;
// 1024 half channels are 8 strips of 256 bytes per row): NR 16-byte vectors
// per thread in registers, NS more in LDS, as in bn_onchip.hip.  A thread's vectors always hold the same VEC channels (the
// strip's width divides 1024), so the per-channel sums are VEC accumulators
// per thread, folded over the block.  The blocks of a strip then exchange
// their per-channel partials as {value, epoch} words (xchg.cuh) in two stages:
// a block merges a few channels over the blocks of their strip (fixed order,
// a group of threads per channel), writes mean / var / running statistics and
// publishes the results in eight copies (block b reads copy b % 8: all blocks
// polling the same words queue up on the memory channel that holds them, a
// copy per block is 256 scattered stores per channel); every block reads its
// copy of its strip's results and normalizes what it holds: x crosses the
// memory system once (2 S).
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

constexpr int kGridMaxBlocks = 256; // blocks of a launch (one per CU)
// Channels of a strip (the per-channel LDS arrays).  Wider strips - up to a
// wave's 64 vectors - were built and lost: the arrays for 512 channels cost
// three LDS slots, and a block's share of the exchange grows with its channels
// ([256,14,14,512] half 29.0 / 47.0 us forward / backward in one strip of 64
// vectors, 26.4 / 43.5 in four of 16; 64-byte strips lose a third).
constexpr int kGridMaxC = 128;
// Copies of the per-channel results of stage 2; block b reads copy b % 8.  A
// copy per block (256 scattered 8-byte stores per channel) made the second hop
// three times as slow as the first, one copy for all makes every block poll the
// same eight cache lines ([256,56,56,64] half forward / backward: 49.1 / 76.0 us
// with 256 copies, 46.9 / 75.0 with 8, 48.4 / 76.0 with one).
constexpr uint32_t kGridCopies = 8;
// Words of the per-block flags: 1024 "partial missing" bits, then "any partial
// missing" and "any result missing".
constexpr int kGridFlagWords = kOnchipBlock / 32 + 2;
constexpr int kGridAnyPartial = kOnchipBlock / 32, kGridAnyResult = kOnchipBlock / 32 + 1;

struct BnClGridArgs {
  const void *x;
  void *y;
  const float *gamma, *beta;
  float *mean, *var, *rmean, *rvar;
  uint32_t C;       // channels of the tensor
  uint32_t ld;      // vectors per row of the tensor = C / VEC
  uint32_t cs;      // channels of a column strip = cv * VEC (the LDS arrays are indexed by the channel within the strip)
  uint32_t cv;      // vectors of a strip's row segment (a power of two, at most 128 channels)
  uint32_t cvsh;    // log2 cv
  uint32_t cssh;    // log2 cs
  uint32_t strips;  // ld / cv; block b holds strip b % strips of row range b / strips
  uint32_t M;       // rows of the tensor
  uint32_t rows_pb; // rows of a range (the last one may have fewer)
  uint32_t ranges;  // row ranges = blocks per strip
  uint32_t nblocks; // ranges * strips
  uint32_t kstep;   // vectors between a thread's consecutive slots = (1024 / cv) * ld
  uint32_t lp;      // stage 2: 2^lp threads per channel, one per block of the strip (2^lp >= ranges)
  uint32_t gu;      // stage 2: channels per block (gu << lp <= 1024)
  uint32_t hv;      // forward: vectors of a block that its threads hold (the rest is streamed), a multiple of 1024
  float inv_N, unbias, decay, eps, one;
  // backward
  const void *dy;
  void *dx;                  // may be null
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;     // may be null
  int accum_dx, accum_g, accum_b;
  unsigned long long *x1; // stage 1: [nblocks][cs][2] = (mean, m2) of the block's rows
                          //          (backward: (sum dy*xh, sum dy))
  unsigned long long *x2; // stage 2: [copies][C][2] = (mean, var)
  uint32_t epoch;
  int spin;
  uint32_t copies; // copies of the stage-2 results; block b reads copy b % copies
};

// Rows of range r.
__device__ __forceinline__ uint32_t grid_range_rows(const BnClGridArgs &a, uint32_t r) {
  const uint32_t first = r * a.rows_pb;
  return first >= a.M ? 0u : min(a.rows_pb, a.M - first);
}

// Vector v of a block (row v / cv of its range, column v % cv of its strip) in
// vectors from the block's first one.  Grows with v.
__device__ __forceinline__ uint32_t grid_offset(const BnClGridArgs &a, uint32_t v) {
  return (v >> a.cvsh) * a.ld + (v & (a.cv - 1u));
}

// First element of block (strip s, range r).
__device__ __forceinline__ size_t grid_block_base(const BnClGridArgs &a, uint32_t s, uint32_t r, int vec) {
  return (static_cast<size_t>(r) * a.rows_pb * a.ld + static_cast<size_t>(s) * a.cv) * vec;
}

// Per-channel totals of v[VEC] over the threads of the block that hold the
// same channel vector (t % cv): butterfly over the lanes cv apart, one row of
// fold[16][cs] per wave, the rows added in wave order by one thread per channel
// (tot[cs]), and every thread reads back its channels' totals.
// (No barrier ahead of the first write: every earlier reader of fold has passed
// the last barrier of the call before, and so has every reader of tot by the
// time tot is written again, two barriers further on.)
template <int VEC>
__device__ __forceinline__ void grid_channel_sums(float (&v)[VEC], uint32_t cv, uint32_t cvx,
                                                  float *fold, float *tot, uint32_t cs) {
  constexpr int NW = kOnchipBlock / kWave;
  lanes_sum_from<VEC>(v, cv); // (a step at a time for all values, off the LDS crossbar: xor_add)
  if ((threadIdx.x & (kWave - 1)) < cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fold[(threadIdx.x / kWave) * cs + cvx * VEC + j] = v[j];
  }
  lds_barrier();
  if (threadIdx.x < cs) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w * cs + threadIdx.x];
    tot[threadIdx.x] = t;
  }
  lds_barrier();
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = tot[cvx * VEC + j];
}

// The same fold for ONE channel (element e of the vectors of channel vector
// cl / VEC of the strip): identical butterfly and wave order, so identical bits.
__device__ __forceinline__ float grid_channel_sum1(float v, uint32_t cv, uint32_t cl, bool mine,
                                                   float *fold, uint32_t cs) {
  constexpr int NW = kOnchipBlock / kWave;
  v = lanes_sum_from(v, cv);
  lds_barrier(); // earlier readers of fold are done
  if ((threadIdx.x & (kWave - 1)) < cv && mine) fold[(threadIdx.x / kWave) * cs + cl] = v;
  lds_barrier();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) t += fold[w * cs + cl];
  return t;
}

// Sum of v over each aligned group of 2^lp consecutive threads, the same value
// in every thread of the group: butterfly over the lanes of a wave, then the
// waves of a group in wave order.  wsum: 16 floats.
__device__ __forceinline__ float grid_group_sum(float v, uint32_t lp, float *wsum) {
  v = lanes_sum_below(v, min(1u << lp, static_cast<uint32_t>(kWave)));
  if (lp > 6) { // (the same in every thread)
    const uint32_t wave = threadIdx.x / kWave, nw = 1u << (lp - 6), w0 = wave & ~(nw - 1u);
    lds_barrier(); // earlier readers of wsum are done
    if ((threadIdx.x & (kWave - 1)) == 0) wsum[wave] = v;
    lds_barrier();
    float s = 0.f;
    for (uint32_t i = 0; i < nw; ++i) s += wsum[w0 + i];
    v = s;
  }
  return v;
}

// (mean, m2) of the rows of block (strip of channel c, range r) for channel c,
// from global memory, in the order that block itself uses (its thread map,
// slots ascending per thread, the thread's own mean as the shift, the same
// folds): what it publishes for c, bit for bit.  Only the threads of c's
// channel vector load (the folds never mix channel vectors) and only c's
// element is accumulated, so this costs a handful of registers.
template <typename T, int VEC>
__device__ __forceinline__ void grid_partial_from_memory(const BnClGridArgs &a, uint32_t r,
                                                         uint32_t c, float *fold, float &m,
                                                         float &q) {
  const uint32_t t = threadIdx.x;
  const uint32_t s = c >> a.cssh, cl = c & (a.cs - 1u);
  const T *__restrict__ x = static_cast<const T *>(a.x) + grid_block_base(a, s, r, VEC);
  const uint32_t cvx = t & (a.cv - 1u), e = cl % VEC;
  const uint32_t vbb = grid_range_rows(a, r) << a.cvsh;
  const bool mine = cvx == cl / VEC;
  const uint32_t vbp = mine ? vbb : 0u;
  const uint32_t vbh = min(vbb, a.hv); // the vectors that block holds: its threads' shifts are their means
  const uint32_t tb = grid_offset(a, t);
  float sx = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll 1
  for (uint32_t v = t, off = tb; v < min(vbp, vbh); v += kOnchipBlock, off += a.kstep) {
    const RawVec<T, VEC> rr = load_raw<T, VEC>(x + static_cast<size_t>(off) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float n = elem_fma<T, VEC>(rr, j, a.one, sx);
      sx = static_cast<uint32_t>(j) == e ? n : sx;
    }
  }
  const float nh = (mine && t < vbh) ? static_cast<float>((vbh - 1u - t) / kOnchipBlock + 1u) : 0.f;
  const float nt = (mine && t < vbb) ? static_cast<float>((vbb - 1u - t) / kOnchipBlock + 1u) : 0.f;
  const float kk = sx * (1.0f / fmaxf(nh, 1.f));
#pragma unroll 1
  for (uint32_t v = t, off = tb; v < vbp; v += kOnchipBlock, off += a.kstep) {
    const RawVec<T, VEC> rr = load_raw<T, VEC>(x + static_cast<size_t>(off) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = elem_fma<T, VEC>(rr, j, a.one, -kk);
      const float n1 = s1 + d;
      const float n2 = fmaf(d, d, s2);
      s1 = static_cast<uint32_t>(j) == e ? n1 : s1;
      s2 = static_cast<uint32_t>(j) == e ? n2 : s2;
    }
  }
  m = grid_channel_sum1(fmaf(nt, kk, s1), a.cv, cl, mine, fold, a.cs);
  m *= 1.0f / static_cast<float>(vbb >> a.cvsh);
  const float d = kk - m;
  q = grid_channel_sum1(mine ? fmaf(d, fmaf(nt, d, 2.f * s1), s2) : 0.f, a.cv, cl, mine, fold, a.cs);
}

// Backward: (sum dy*xh, sum dy) of the rows of block (strip of c, range r) for
// channel c, from global memory, in that block's own order (slots ascending
// per thread, the same folds): what it publishes for c, bit for bit.
template <typename T, int VEC>
__device__ __forceinline__ void grid_pair_from_memory(const BnClGridArgs &a, uint32_t r,
                                                      uint32_t c, float *fold, float &sdx,
                                                      float &sdy) {
  const uint32_t t = threadIdx.x;
  const uint32_t s = c >> a.cssh, cl = c & (a.cs - 1u);
  const size_t base = grid_block_base(a, s, r, VEC);
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + base;
  const uint32_t cvx = t & (a.cv - 1u), e = cl % VEC;
  const bool mine = cvx == cl / VEC;
  const uint32_t vbp = mine ? grid_range_rows(a, r) << a.cvsh : 0u;
  const float mean = a.mean[c];
  const float istd = 1.0f / sqrtf(a.var[c] + a.eps);
  const float nmi = -mean * istd;
  sdx = 0.f;
  sdy = 0.f;
#pragma unroll 1
  for (uint32_t v = t, off = grid_offset(a, t); v < vbp; v += kOnchipBlock, off += a.kstep) {
    const RawVec<T, VEC> xr = load_raw<T, VEC>(x + static_cast<size_t>(off) * VEC);
    const RawVec<T, VEC> dr = load_raw<T, VEC>(dy + static_cast<size_t>(off) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr, j, mean, istd, nmi);
      const float nx = elem_fma<T, VEC>(dr, j, xh, sdx);
      const float ny = elem_fma<T, VEC>(dr, j, a.one, sdy);
      sdx = static_cast<uint32_t>(j) == e ? nx : sdx;
      sdy = static_cast<uint32_t>(j) == e ? ny : sdy;
    }
  }
  sdx = grid_channel_sum1(sdx, a.cv, cl, mine, fold, a.cs);
  sdy = grid_channel_sum1(sdy, a.cv, cl, mine, fold, a.cs);
}

// Stage 2 of both directions: the partials of `count` channels from `cfirst`
// on, one channel per group of 2^lp threads, thread p of a group taking the
// partial of block (strip of the channel, range p) - polled; computed here,
// by the whole block, if it does not arrive.  v0 / v1 are the two words of the
// partial (0 in a thread without one).  flags: kGridFlagWords words.
template <typename T, int VEC, bool BWD>
__device__ __forceinline__ void grid_collect(const BnClGridArgs &a, uint32_t cfirst, uint32_t count,
                                             uint32_t *flags, float *fold, float &v0, float &v1) {
  const uint32_t t = threadIdx.x;
  const uint32_t g = t >> a.lp, p = t & ((1u << a.lp) - 1u);
  lds_barrier(); // the flags of an earlier call have been consumed
  if (t <= static_cast<uint32_t>(kGridAnyPartial)) flags[t] = 0;
  lds_barrier();
  v0 = 0.f;
  v1 = 0.f;
  if (g < count && p < a.ranges) {
    const uint32_t c = cfirst + g;
    const uint32_t bp = p * a.strips + (c >> a.cssh);
    const bool ok = xchg_poll2(a.x1 + (static_cast<size_t>(bp) * a.cs + (c & (a.cs - 1u))) * 2, a.epoch,
                               a.spin, &v0, &v1);
    if (!ok) {
      atomicOr(&flags[t >> 5], 1u << (t & 31u));
      flags[kGridAnyPartial] = 1;
    }
  }
  lds_barrier();
  if (flags[kGridAnyPartial] == 0) return; // (the same in every thread)
  for (uint32_t w = 0; w < static_cast<uint32_t>(kOnchipBlock / 32); ++w) {
    uint32_t bits = __builtin_amdgcn_readfirstlane(flags[w]);
    while (bits) {
      const uint32_t idx = w * 32u + static_cast<uint32_t>(__builtin_ctz(bits));
      bits &= bits - 1u;
      float r0, r1;
      if constexpr (BWD) {
        grid_pair_from_memory<T, VEC>(a, idx & ((1u << a.lp) - 1u), cfirst + (idx >> a.lp), fold, r0, r1);
      } else {
        grid_partial_from_memory<T, VEC>(a, idx & ((1u << a.lp) - 1u), cfirst + (idx >> a.lp), fold, r0, r1);
      }
      if (t == idx) {
        v0 = r0;
        v1 = r1;
      }
    }
  }
}

// Merged (mean, var) of `count` channels from `cfirst` on over the blocks of
// their strips: mean = sum n_p * mean_p / N, m2 = sum (m2_p + n_p * (mean_p -
// mean)^2), two group sums in a fixed order (a Chan merge tree over 256
// partials took 2.5 us).  The threads of group g return channel cfirst + g;
// same result in every block that calls it, whatever else it merges alongside.
template <typename T, int VEC>
__device__ __forceinline__ void grid_channel_result(const BnClGridArgs &a, uint32_t cfirst,
                                                    uint32_t count, uint32_t *flags, float *wsum,
                                                    float *fold, float &mean, float &var) {
  float mp, qp;
  grid_collect<T, VEC, false>(a, cfirst, count, flags, fold, mp, qp);
  const uint32_t t = threadIdx.x;
  const uint32_t g = t >> a.lp, p = t & ((1u << a.lp) - 1u);
  const float np = (g < count && p < a.ranges) ? static_cast<float>(grid_range_rows(a, p)) : 0.f;
  mean = grid_group_sum(np * mp, a.lp, wsum) * a.inv_N;
  const float d = mp - mean;
  var = grid_group_sum(fmaf(np * d, d, qp), a.lp, wsum) * a.inv_N;
}

// Backward: (sum dy*xh, sum dy) of `count` channels from `cfirst` on over the
// blocks of their strips, in block order.
template <typename T, int VEC>
__device__ __forceinline__ void grid_pair_result(const BnClGridArgs &a, uint32_t cfirst, uint32_t count,
                                                 uint32_t *flags, float *wsum, float *fold, float &sdx,
                                                 float &sdy) {
  float px, py;
  grid_collect<T, VEC, true>(a, cfirst, count, flags, fold, px, py);
  sdx = grid_group_sum(px, a.lp, wsum);
  sdy = grid_group_sum(py, a.lp, wsum);
}

} // namespace

// OVER: the block has more vectors than the NR + NS its threads hold; the rest
// is read for the statistics and again for the normalization.
template <typename T, int VEC, int NR, int NS, bool OVER>
__global__ void __launch_bounds__(kOnchipBlock)
bn_cl_grid_fwd_kernel(const BnClGridArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  constexpr int CMAX = kGridMaxC;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float fold[16 * CMAX];
  __shared__ float tot[CMAX];
  __shared__ float fin[2 * CMAX];   // (mean, var) per channel of the strip
  __shared__ uint32_t flags[kGridFlagWords];
  __shared__ float wsum[16];
  __shared__ float gb[2 * CMAX]; // gamma, beta
  const uint32_t b = blockIdx.x;
  const uint32_t t = threadIdx.x;
  const uint32_t strip = b % a.strips, range = b / a.strips;
  const uint32_t c0 = strip << a.cssh; // the strip's first channel
  // gamma and beta of channel t of the strip, asked for ahead of the tensor
  // (behind the exchange they would cost a memory round trip of their own)
  float gamma_t = 1.f, beta_t = 0.f;
  if (t < a.cs) {
    if (a.gamma) gamma_t = a.gamma[c0 + t];
    if (a.beta) beta_t = a.beta[c0 + t];
  }
  const uint32_t cvx = t & (a.cv - 1u);
  const uint32_t ch = cvx * VEC;
  const uint32_t vbb = grid_range_rows(a, range) << a.cvsh;
  const size_t base = grid_block_base(a, strip, range, VEC);
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  T *__restrict__ y = static_cast<T *>(a.y) + base;

  // ---- loads: slot k is vector k * 1024 + t of the block, at tb + k * kstep
  // (a slot past the block's end reads the block's last vector and stays out
  // of sums and stores)
  const uint32_t tb = grid_offset(a, t);
  const uint32_t last = grid_offset(a, vbb - 1u);
  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t o = tb + static_cast<uint32_t>(NR + k) * a.kstep;
      parked[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(o, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t o = tb + static_cast<uint32_t>(k) * a.kstep;
      raw[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(o, last)) * VEC);
    }
    if (t < a.cs) { // (they arrive first; read behind the barriers of the folds)
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

  // (slot k holds a vector of the block: an offset against a scalar, no register per slot)
  auto holds = [&](int k) {
    return static_cast<int>(tb) <= static_cast<int>(last) - k * static_cast<int>(a.kstep);
  };

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
  // (The thread's sum enters the mean as n K + s1.  What a block streams, OVER,
  // is taken about the K of the vectors held: K is then not the thread's mean
  // but close to it, s1 no longer a residue, and the same formulas hold.)
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
    const uint32_t vbh = OVER ? min(vbb, static_cast<uint32_t>(NL) * kOnchipBlock) : vbb;
    const float nh = t < vbh ? static_cast<float>((vbh - 1u - t) / kOnchipBlock + 1u) : 0.f;
    const float nt = t < vbb ? static_cast<float>((vbb - 1u - t) / kOnchipBlock + 1u) : 0.f;
    const float rnt = 1.0f / fmaxf(nh, 1.f);
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
    if constexpr (OVER) { // two vectors in flight
#pragma unroll 1
      for (uint32_t o = tb + static_cast<uint32_t>(NL) * a.kstep; o <= last; o += 2 * a.kstep) {
        const uint32_t o1 = o + a.kstep;
        const RawVec<T, VEC> r0 = load_raw<T, VEC>(x + static_cast<size_t>(o) * VEC);
        const RawVec<T, VEC> r1 = load_raw<T, VEC>(x + static_cast<size_t>(min(o1, last)) * VEC);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(r0, j, a.one, -kk[j]);
          s1[j] += d;
          s2[j] = fmaf(d, d, s2[j]);
        }
        if (o1 <= last) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float d = elem_fma<T, VEC>(r1, j, a.one, -kk[j]);
            s1[j] += d;
            s2[j] = fmaf(d, d, s2[j]);
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) m[j] = fmaf(nt, kk[j], s1[j]);
    grid_channel_sums<VEC>(m, a.cv, cvx, fold, tot, a.cs);
    const float icnt = 1.0f / static_cast<float>(vbb >> a.cvsh);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      m[j] *= icnt;
      const float e = kk[j] - m[j];
      q[j] = fmaf(e, fmaf(nt, e, 2.f * s1[j]), s2[j]);
    }
    grid_channel_sums<VEC>(q, a.cv, cvx, fold, tot, a.cs);
  }
  // publish (mean, m2) of every channel of the strip: a word per thread
  // (through fin, which is free until the results arrive)
  if (t < a.cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      fin[2 * (ch + j)] = m[j];
      fin[2 * (ch + j) + 1] = q[j];
    }
  }
  lds_barrier();
  for (uint32_t e = t; e < 2 * a.cs; e += kOnchipBlock)
    xchg_publish(a.x1 + static_cast<size_t>(b) * a.cs * 2 + e, fin[e], a.epoch);

  // ---- stage 2: block b merges channels b * gu ..., writes their statistics, publishes
  if (const uint32_t cfirst = b * a.gu; cfirst < a.C) {
    const uint32_t count = min(a.gu, a.C - cfirst);
    float mean, var;
    grid_channel_result<T, VEC>(a, cfirst, count, flags, wsum, fold, mean, var);
    const uint32_t g = t >> a.lp, p = t & ((1u << a.lp) - 1u);
    if (g < count) {
      const uint32_t c = cfirst + g;
      if (p == 0) {
        a.mean[c] = mean;
        a.var[c] = var;
        if (a.rmean) a.rmean[c] = a.decay * a.rmean[c] + (1.f - a.decay) * mean;
        if (a.rvar) a.rvar[c] = a.decay * a.rvar[c] + (1.f - a.decay) * var * a.unbias;
      }
      if (p < a.copies) { // copy p
        unsigned long long *w = a.x2 + (static_cast<size_t>(p) * a.C + c) * 2;
        xchg_publish(w, mean, a.epoch);
        xchg_publish(w + 1, var, a.epoch);
      }
    }
  }

  // ---- every block: the results of its strip (merged here where one does not arrive)
  lds_barrier();
  if (t == 0) flags[kGridAnyResult] = 0;
  lds_barrier();
  for (uint32_t c = t; c < a.cs; c += kOnchipBlock) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x2 + (static_cast<size_t>(b % a.copies) * a.C + c0 + c) * 2, a.epoch,
                               a.spin, &v0, &v1);
    fin[2 * c] = v0;
    fin[2 * c + 1] = ok ? v1 : -1.f; // a variance is never negative: marks "missing"
    if (!ok) flags[kGridAnyResult] = 1;
  }
  lds_barrier();
  for (uint32_t c = 0; flags[kGridAnyResult] && c < a.cs; ++c) {
    if (fin[2 * c + 1] >= 0.f) continue; // same answer in every thread
    float mean, var;
    grid_channel_result<T, VEC>(a, c0 + c, 1u, flags, wsum, fold, mean, var);
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
  // (scale and shift of a channel by one thread, through fold, which is free
  // now: 1 / sqrt once per channel instead of VEC times in every thread,
  // behind the exchange where every instruction is on the critical path)
  if (t < a.cs) {
    const float scale = gb[t] * inv_std(fin[2 * t + 1], a.eps);
    fold[t] = scale;
    fold[CMAX + t] = fmaf(-fin[2 * t], scale, gb[CMAX + t]);
  }
  lds_barrier();
  float sc[VEC], sh[VEC], mu[VEC], be[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mu[j] = fin[2 * (ch + j)];
    sc[j] = fold[ch + j];
    be[j] = gb[CMAX + ch + j];
    sh[j] = fold[CMAX + ch + j];
  }
  const uint32_t tb2 = grid_offset(a, fresh(t));
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t o = tb2 + static_cast<uint32_t>(k) * a.kstep;
    if (o <= last) {
      const RawVec<T, VEC> r = slot(k);
      float ov[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          ov[j] = elem_fma<T, VEC>(r, j, sc[j], sh[j]);
        } else {
          ov[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mu[j]), sc[j], be[j]);
        }
      }
      store_vec<T, VEC>(y + static_cast<size_t>(o) * VEC, ov);
    }
  }
  if constexpr (OVER) {
    auto emit = [&](const RawVec<T, VEC> &r, uint32_t o) {
      float ov[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          ov[j] = elem_fma<T, VEC>(r, j, sc[j], sh[j]);
        } else {
          ov[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mu[j]), sc[j], be[j]);
        }
      }
      store_vec<T, VEC>(y + static_cast<size_t>(o) * VEC, ov);
    };
#pragma unroll 1
    for (uint32_t o = tb2 + static_cast<uint32_t>(NL) * a.kstep; o <= last; o += 2 * a.kstep) {
      const uint32_t o1 = o + a.kstep;
      const RawVec<T, VEC> r0 = load_raw<T, VEC>(x + static_cast<size_t>(o) * VEC);
      const RawVec<T, VEC> r1 = load_raw<T, VEC>(x + static_cast<size_t>(min(o1, last)) * VEC);
      emit(r0, o);
      if (o1 <= last) emit(r1, o1);
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
// forward's two stages, the merging block writing dgamma / dbeta.
template <typename T, int VEC, int NR, int NS, int B>
__global__ void __launch_bounds__(kOnchipBlock)
bn_cl_grid_bwd_kernel(const BnClGridArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  constexpr int CMAX = kGridMaxC;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float fold[16 * CMAX];
  __shared__ float tot[CMAX];
  __shared__ float fin[2 * CMAX]; // (sdx, sdy) totals per channel of the strip
  __shared__ int finmiss[CMAX];
  __shared__ uint32_t flags[kGridFlagWords];
  __shared__ float wsum[16];
  __shared__ float par[6 * CMAX]; // mean, var, gamma, dvar, dmean, istd
  const uint32_t b = blockIdx.x;
  const uint32_t t = threadIdx.x;
  const uint32_t strip = b % a.strips, range = b / a.strips;
  const uint32_t c0 = strip << a.cssh;
  // The parameters of channel t of the strip, asked for ahead of the tensor:
  // behind the LDS stores of x, or behind the exchange, each would cost a
  // memory round trip of its own.
  float p_mean = 0.f, p_var = 1.f, p_gamma = 1.f, p_dvar = 0.f, p_dmean = 0.f;
  if (t < a.cs) {
    p_mean = a.mean[c0 + t];
    p_var = a.var[c0 + t];
    if (a.gamma) p_gamma = a.gamma[c0 + t];
    if (a.dvar) p_dvar = a.dvar[c0 + t];
    if (a.dmean) p_dmean = a.dmean[c0 + t];
  }
  const uint32_t cvx = t & (a.cv - 1u);
  const uint32_t ch = cvx * VEC;
  const uint32_t vbb = grid_range_rows(a, range) << a.cvsh;
  const size_t base = grid_block_base(a, strip, range, VEC);
  const T *__restrict__ x = static_cast<const T *>(a.x) + base;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + base;
  T *__restrict__ dx = a.dx ? static_cast<T *>(a.dx) + base : nullptr;
  const uint32_t last = grid_offset(a, vbb - 1u);

  RawVec<T, VEC> raw[NR];
  {
    const uint32_t tb = grid_offset(a, t);
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t o = tb + static_cast<uint32_t>(NR + k) * a.kstep;
      parked[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(o, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t o = tb + static_cast<uint32_t>(k) * a.kstep;
      raw[k] = load_raw<T, VEC>(x + static_cast<size_t>(min(o, last)) * VEC);
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };
  if (t < a.cs) {
    par[t] = p_mean;
    par[CMAX + t] = p_var;
    par[2 * CMAX + t] = p_gamma;
    par[3 * CMAX + t] = p_dvar;
    par[4 * CMAX + t] = p_dmean;
    par[5 * CMAX + t] = 1.0f / sqrtf(p_var + a.eps);
  }
  lds_barrier();
  float mean[VEC], istd[VEC], nmi[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mean[j] = par[ch + j];
    istd[j] = par[5 * CMAX + ch + j];
    nmi[j] = -mean[j] * istd[j];
  }

  // ---- pass 1: the block's (sum dy*xh, sum dy) per channel, vectors ascending
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t tb1 = grid_offset(a, fresh_after(t, sdx[0]));
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const uint32_t o = tb1 + static_cast<uint32_t>(k0 + i) * a.kstep;
      d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(o, last)) * VEC);
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      if (k < NL && tb1 + static_cast<uint32_t>(k) * a.kstep <= last) {
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
  // (what the block does not hold: x and dy streamed, two vectors of each in flight)
#pragma unroll 1
  for (uint32_t o = grid_offset(a, fresh_after(t, sdx[0])) + static_cast<uint32_t>(NL) * a.kstep; o <= last;
       o += 2 * a.kstep) {
    const uint32_t o1 = o + a.kstep;
    const RawVec<T, VEC> xr0 = load_raw<T, VEC>(x + static_cast<size_t>(o) * VEC);
    const RawVec<T, VEC> dr0 = load_raw<T, VEC>(dy + static_cast<size_t>(o) * VEC);
    const RawVec<T, VEC> xr1 = load_raw<T, VEC>(x + static_cast<size_t>(min(o1, last)) * VEC);
    const RawVec<T, VEC> dr1 = load_raw<T, VEC>(dy + static_cast<size_t>(min(o1, last)) * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xh = norm_elem<T, VEC>(xr0, j, mean[j], istd[j], nmi[j]);
      sdx[j] = elem_fma<T, VEC>(dr0, j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dr0, j, a.one, sdy[j]);
    }
    if (o1 <= last) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr1, j, mean[j], istd[j], nmi[j]);
        sdx[j] = elem_fma<T, VEC>(dr1, j, xh, sdx[j]);
        sdy[j] = elem_fma<T, VEC>(dr1, j, a.one, sdy[j]);
      }
    }
  }
  grid_channel_sums<VEC>(sdx, a.cv, cvx, fold, tot, a.cs);
  if (t < a.cv) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fin[ch + j] = sdx[j];
  }
  grid_channel_sums<VEC>(sdy, a.cv, cvx, fold, tot, a.cs);
  // (fin's stores precede the barriers of the second fold: visible by now)
  for (uint32_t e = t; e < 2 * a.cs; e += kOnchipBlock)
    xchg_publish(a.x1 + static_cast<size_t>(b) * a.cs * 2 + e, (e & 1) ? tot[e >> 1] : fin[e >> 1], a.epoch);

  // ---- stage 2: block b sums channels b * gu ... over the blocks of their
  // strips, writes dgamma / dbeta, publishes
  if (const uint32_t cfirst = b * a.gu; cfirst < a.C) {
    const uint32_t count = min(a.gu, a.C - cfirst);
    float tx, ty;
    grid_pair_result<T, VEC>(a, cfirst, count, flags, wsum, fold, tx, ty);
    const uint32_t g = t >> a.lp, p = t & ((1u << a.lp) - 1u);
    if (g < count) {
      const uint32_t c = cfirst + g;
      if (p == 0) {
        if (a.dgamma) a.dgamma[c] = tx + (a.accum_g ? a.dgamma[c] : 0.f);
        if (a.dbeta) a.dbeta[c] = ty + (a.accum_b ? a.dbeta[c] : 0.f);
      }
      if (p < a.copies) { // copy p
        unsigned long long *w = a.x2 + (static_cast<size_t>(p) * a.C + c) * 2;
        xchg_publish(w, tx, a.epoch);
        xchg_publish(w + 1, ty, a.epoch);
      }
    }
  }
  if (dx == nullptr) return;

  // ---- every block: the totals of its strip (summed here where one does not arrive)
  lds_barrier();
  if (t == 0) flags[kGridAnyResult] = 0;
  lds_barrier();
  for (uint32_t c = t; c < a.cs; c += kOnchipBlock) {
    float v0 = 0.f, v1 = 0.f;
    const bool ok = xchg_poll2(a.x2 + (static_cast<size_t>(b % a.copies) * a.C + c0 + c) * 2, a.epoch,
                               a.spin, &v0, &v1);
    fin[2 * c] = v0;
    fin[2 * c + 1] = v1;
    finmiss[c] = ok ? 0 : 1;
    if (!ok) flags[kGridAnyResult] = 1;
  }
  lds_barrier();
  for (uint32_t c = 0; flags[kGridAnyResult] && c < a.cs; ++c) {
    if (!finmiss[c]) continue; // same answer in every thread
    float tx, ty;
    grid_pair_result<T, VEC>(a, c0 + c, 1u, flags, wsum, fold, tx, ty);
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
  // The coefficients of a channel by one thread, through fold, which is free
  // now (behind the exchange every instruction is on the critical path); the
  // means from LDS again: kept in registers across the exchange, they and the
  // vectors of x are more than a thread has.
  if (t < a.cs) {
    const float g = par[2 * CMAX + t];
    const float vpe = par[CMAX + t] + a.eps;
    const float is = par[5 * CMAX + t];
    const float cA = -is * g * fin[2 * t] * a.inv_N +
                     (a.dvar ? 2.f * par[3 * CMAX + t] * (vpe * is) * a.inv_N : 0.f);
    const float cb = -g * fin[2 * t + 1] * is * a.inv_N + (a.dmean ? par[4 * CMAX + t] * a.inv_N : 0.f);
    fold[t] = g * is;
    fold[CMAX + t] = is * cA;
    fold[2 * CMAX + t] = sizeof(T) == 2 ? fmaf(-par[t] * is, cA, cb) : cb;
  }
  lds_barrier();
  float gi[VEC], A2[VEC], B2[VEC], mean2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    mean2[j] = par[ch + j];
    gi[j] = fold[ch + j];
    A2[j] = fold[CMAX + ch + j];
    B2[j] = fold[2 * CMAX + ch + j];
  }
  auto emit = [&](const RawVec<T, VEC> &xr, const RawVec<T, VEC> &dr, uint32_t o) {
    float ov[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float xt;
      if constexpr (sizeof(T) == 2) {
        xt = elem_fma<T, VEC>(xr, j, A2[j], B2[j]);
      } else {
        xt = fmaf(elem_fma<T, VEC>(xr, j, a.one, -mean2[j]), A2[j], B2[j]);
      }
      ov[j] = elem_fma<T, VEC>(dr, j, gi[j], xt);
    }
    T *dst = dx + static_cast<size_t>(o) * VEC;
    if (a.accum_dx) {
      float old[VEC];
      load_vec<T, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) ov[j] += old[j];
    }
    store_vec<T, VEC>(dst, ov);
  };
  float lastv = B2[0];
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t tb2 = grid_offset(a, fresh_after(t, lastv));
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const uint32_t o = tb2 + static_cast<uint32_t>(k0 + i) * a.kstep;
      d[i] = load_raw<T, VEC>(dy + static_cast<size_t>(min(o, last)) * VEC);
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const int k = k0 + i;
      const uint32_t o = tb2 + static_cast<uint32_t>(k) * a.kstep;
      if (k < NL && o <= last) {
        emit(slot(k), d[i], o);
        lastv = __builtin_bit_cast(float, __builtin_bit_cast(uint4, d[i]).x);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll 1
  for (uint32_t o = grid_offset(a, fresh_after(t, lastv)) + static_cast<uint32_t>(NL) * a.kstep; o <= last;
       o += 2 * a.kstep) {
    const uint32_t o1 = o + a.kstep;
    const RawVec<T, VEC> xr0 = load_raw<T, VEC>(x + static_cast<size_t>(o) * VEC);
    const RawVec<T, VEC> dr0 = load_raw<T, VEC>(dy + static_cast<size_t>(o) * VEC);
    const RawVec<T, VEC> xr1 = load_raw<T, VEC>(x + static_cast<size_t>(min(o1, last)) * VEC);
    const RawVec<T, VEC> dr1 = load_raw<T, VEC>(dy + static_cast<size_t>(min(o1, last)) * VEC);
    emit(xr0, dr0, o);
    if (o1 <= last) emit(xr1, dr1, o1);
  }
}

namespace {

template <typename T, int VEC>
int run_grid_fwd(int nl, const BnClGridArgs &a, hipStream_t st) {
#define GRID_CASE(NR, NS)                                                                        \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH("bn_cl_grid_fwd_kernel", (bn_cl_grid_fwd_kernel<T, VEC, NR, NS, false>),      \
                   dim3(a.nblocks), dim3(kOnchipBlock), 0, st, a);                               \
    return last_launch_status();                                                                 \
  }
  GRID_CASE(4, 0)
  GRID_CASE(8, 0)
  GRID_CASE(12, 0)
  GRID_CASE(16, 0)
  GRID_CASE(16, 3)
  GRID_CASE(16, 6)
  GRID_CASE(16, 9)
#undef GRID_CASE
  // (more per thread than the 25 vectors held: the rest is read twice)
  NBLAHIP_LAUNCH("bn_cl_grid_fwd_kernel", (bn_cl_grid_fwd_kernel<T, VEC, 16, 9, true>), dim3(a.nblocks),
                 dim3(kOnchipBlock), 0, st, a);
  return last_launch_status();
}

template <typename T, int VEC>
int run_grid_bwd(int nl, const BnClGridArgs &a, hipStream_t st) {
  constexpr int B = sizeof(T) == 2 ? 2 : 4;
#define GRID_CASE(NR, NS)                                                                        \
  if (nl <= (NR) + (NS)) {                                                                       \
    constexpr int kNS = (NS) > 9 ? 9 : (NS);                                                     \
    NBLAHIP_LAUNCH("bn_cl_grid_bwd_kernel", (bn_cl_grid_bwd_kernel<T, VEC, NR, kNS, B>),         \
                   dim3(a.nblocks), dim3(kOnchipBlock), 0, st, a);                               \
    return last_launch_status();                                                                 \
  }
  GRID_CASE(4, 0)
  GRID_CASE(8, 0)
  GRID_CASE(12, 0)
  GRID_CASE(12, 3)
  GRID_CASE(12, 6)
  // (more per thread than the 21 vectors held: the rest is streamed with dy)
  GRID_CASE(12, 1 << 20)
#undef GRID_CASE
  return NBLAHIP_EINVAL;
}

constexpr int kGridMaxSlots = 25; // vectors per thread the forward layouts hold
constexpr int kGridBwdHeld = 21;  // ... and the backward layouts (12 in registers, 9 in LDS)

int log2_of(uint32_t v) {
  int s = 0;
  while ((1u << s) < v) ++s;
  return s;
}

// Shape test and the arguments both directions share; nl = vectors per thread.
bool grid_args(const BnProblem &p, BnClGridArgs &a, int &nl) {
  if (!tune_int("BN_CL_GRID", 1)) return false;
  if (p.size2 != 1 || p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.C % vec != 0 || !aligned16(p.x) || (p.out && !aligned16(p.out))) return false;
  const int64_t M = p.size0;
  const int64_t ld = p.C / vec;
  if (ld > 4096 || M >= (int64_t{1} << 31)) return false;
  // A block whose partner's word does not arrive reads the partner's rows of x
  // (and dy) again, which the partner may already be overwriting in place.
  const uint64_t tensor_bytes = static_cast<uint64_t>(M * p.C) * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (ranges_overlap(p.out, p.x, tensor_bytes) || ranges_overlap(p.out, p.dy, tensor_bytes)) return false;

  // Column strips: the widest power of two of vectors that divides a row, up
  // to 128 channels.  One strip: the block's rows are contiguous memory.
  // (fewer blocks than CUs: for tests of the streamed remainder on small tensors)
  const int blocks = std::max(8, std::min({device_cus(), kGridMaxBlocks, tune_int("BN_CL_GRID_BLOCKS", kGridMaxBlocks)}));
  int64_t cv = std::min<int64_t>(ld & -ld, kGridMaxC / vec);
  for (const int64_t cap = tune_int("BN_CL_GRID_STRIP_VECS", kWave); cv > cap && cv > 1;) cv >>= 1;
  const int64_t strips = ld / cv;
  if (strips > 1) {
    // (a strip's row segment is at least half a cache line; the callers take
    // the halves only for tensors the chip holds whole)
    if (!tune_int("BN_CL_GRID_STRIPS", 1) || cv < tune_int("BN_CL_GRID_STRIP_MIN_VECS", 4)) return false;
    if (strips > blocks / 8) return false;
  }
  int64_t ranges = std::max<int64_t>(blocks / strips, 1);
  // whole rows per block, the same for every block but the last of a strip
  const int64_t rows_pb = (M + ranges - 1) / ranges;
  nl = static_cast<int>((rows_pb * cv + kOnchipBlock - 1) / kOnchipBlock);
  ranges = (M + rows_pb - 1) / rows_pb;
  // From the rows on below which the split kernels (a block per 1024 rows) are
  // as fast or faster.  Forward + backward us from HBM, this against the split
  // kernels (or, beyond what those take, the split reduction).  Up to 128
  // channels, half [M, 64]: 22.8 vs 21.9 at M = 6272, 23.1 vs 29.1 at 12544,
  // 24.8 vs 32.9 at 50176, 33.6 vs 55.0 at 150528; float 19.5 vs 18.6, 20.0 vs
  // 22.2, 24.2 vs 31.5.  More channels (column strips), half: [6272,256] 22.5 vs
  // 24.3, [12544,256] 24.7 vs 31.7, [12544,512] 28.6 vs 34.6, [6272,1024] 27.9 vs
  // 28.9, [12544,1024] 38.3 vs 40.8, [25088,1024] 65.1 vs 97.0, [6272,2048] 37.2
  // vs 41.7, [3136,4096] 36.8 vs 40.2; float [12544,256] 27.1 vs 30.9,
  // [6272,1024] 35.4 vs 37.5, [12544,1024] 62.0 vs 77.6, [3136,2048] 34.5 vs
  // 36.5; but [3136,256] half 22.2 vs 21.5, [3136,512] float 21.6 vs 20.4: from
  // 10240 rows ([8192,128] float 20.6 vs 17.5) or, with more than 128 channels,
  // 24 MiB.
  // (Rows that are no whole number of 128-byte segments: no split kernel takes
  // them, the other plan is three launches, and these kernels are ahead from the
  // first tensor they accept - forward / backward us, [N,14,14,C] half: 1568 rows
  // of 480 channels 13.7 / 13.0 -> 10.0 / 10.7, 3136 of 96 13.0 / 13.2 -> 10.4 /
  // 11.2, 6272 of 672 19.2 / 21.3 -> 12.9 / 14.8; float 3136 of 80 12.7 / 13.2 ->
  // 8.9 / 9.2.)
  if (p.C % (8 * vec) != 0) {
    if (M < tune_int("BN_CL_GRID_NARROW_MIN_ROWS", 1)) return false;
  } else if (p.C <= kGridMaxC) {
    if (M < tune_int("BN_CL_GRID_MIN_ROWS", 10240)) return false;
  } else {
    if (!tune_int("BN_CL_GRID_WIDE", 1)) return false;
    if (M < tune_int("BN_CL_GRID_WIDE_MIN_ROWS", 10240) &&
        tensor_bytes < static_cast<uint64_t>(tune_int("BN_CL_GRID_WIDE_MIN_KB", 24576)) * 1024u)
      return false;
  }
  const int64_t nblocks = ranges * strips;
  if (nl < tune_int("BN_CL_GRID_MIN_SLOTS", 1) || nblocks < blocks / 2) return false;
  const int lp = log2_of(static_cast<uint32_t>(ranges));
  const int64_t gu = (p.C + nblocks - 1) / nblocks;
  if ((gu << lp) > kOnchipBlock) return false;
  a = BnClGridArgs{};
  a.x = p.x;
  a.gamma = p.gamma;
  a.C = static_cast<uint32_t>(p.C);
  a.ld = static_cast<uint32_t>(ld);
  a.cv = static_cast<uint32_t>(cv);
  a.cs = static_cast<uint32_t>(cv * vec);
  a.cvsh = static_cast<uint32_t>(log2_of(a.cv));
  a.cssh = static_cast<uint32_t>(log2_of(a.cs));
  a.strips = static_cast<uint32_t>(strips);
  a.M = static_cast<uint32_t>(M);
  a.rows_pb = static_cast<uint32_t>(rows_pb);
  a.ranges = static_cast<uint32_t>(ranges);
  a.nblocks = static_cast<uint32_t>(nblocks);
  a.kstep = static_cast<uint32_t>((kOnchipBlock / cv) * ld);
  a.lp = static_cast<uint32_t>(lp);
  a.gu = static_cast<uint32_t>(gu);
  const double N = static_cast<double>(M);
  a.inv_N = static_cast<float>(1.0 / N);
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  a.spin = tune_int("XCHG_SPIN", 64) * 16; // a whole-chip exchange: wait longer before recomputing
  a.copies = std::min<uint32_t>(kGridCopies, a.ranges);
  return true;
}

// Exchange words of both stages.
bool grid_exchange(const BnProblem &p, BnClGridArgs &a, hipStream_t st, int *status) {
  const size_t w1 = static_cast<size_t>(a.nblocks) * a.cs * 2;
  const size_t words = w1 + static_cast<size_t>(a.copies) * p.C * 2;
  if (!xchg_acquire(words, st, &a.x1, &a.epoch, status)) return false;
  a.x2 = a.x1 + w1;
  return true;
}

} // namespace

bool bn_cl_grid_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnClGridArgs a;
  int nl = 0;
  if (!p.out || !grid_args(p, a, nl)) return false;
  // More than the 25 vectors per thread held: the rest is read twice, 2 S for
  // what is held and 3 S for the rest in one launch against 3 S in three
  // ([256,28,28,384] half, 154 MB, 37 vectors: 92.4 -> 67.9 us; 205 MB: 113.7 ->
  // 93.6; 308 MB, 74 vectors: 166.2 -> 150.3; 411 MB, 98 vectors: 223.4 -> 220.9).
  if (nl > tune_int("BN_CL_GRID_FWD_MAX_SLOTS", 80)) return false;
  // Strips of 64 bytes (rows that are no whole number of 128-byte segments: 96,
  // 160, 480, 672 half channels) share their cache lines with the neighbouring
  // strip's blocks: ahead of the three launches where every vector is held
  // (half forward / backward us, [128,14,14,672] 33.5 / 57.4 -> 24.3 / 40.1,
  // [64,56,56,96] 32.1 / 54.5 -> 28.4 / 46.7, [128,28,28,480] forward 64.3 -> 59.6),
  // behind them where a remainder is streamed ([256,28,28,288] backward 104.7 ->
  // 133.6, [128,28,28,480] backward 90.7 -> 102.3).
  if (a.cv < 8 && nl > kGridMaxSlots) return false;
  a.hv = nl > kGridMaxSlots ? static_cast<uint32_t>(kGridMaxSlots) * kOnchipBlock : ~0u;
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
  // Beyond the 21 vectors per thread a block holds, x is read twice like dy: 4 S
  // for what is held and 5 S for the rest in one launch against 5 S in three
  // ([256,28,28,384] half, 154 MB: 138.7 -> 116.9 us; 205 MB half 182.5 ->
  // 179.6, float 189.7 -> 166.4; 257 MB, 62 vectors: 220.4 -> 227.6).
  if (!aligned16(p.dy) || nl > tune_int("BN_CL_GRID_BWD_MAX_SLOTS", 50)) return false;
  // (64-byte strips, see the forward: backward only up to 56 MiB in half, 16 MiB
  // in float - us, this against the three launches, [N,28,28,C]: half C = 96
  // 24 MiB 33.2 / 37.8, 48 MiB 57.4 / 68.1, 64 MiB 73.3 / 68.7; C = 288 48 MiB
  // 55.0 / 79.4, 80 MiB 85.7 / 85.2; float C = 80 12 MiB 17.2 / 18.2, 24 MiB
  // 31.0 / 27.8, 48 MiB 55.0 / 47.1)
  if (a.cv < 8) {
    const uint64_t bytes = static_cast<uint64_t>(p.size0) * p.C * (p.dtype == NBLAHIP_F16 ? 2 : 4);
    const int most_kb = p.dtype == NBLAHIP_F16 ? tune_int("BN_CL_GRID_NARROW_BWD_MAX_KB", 57344)
                                               : tune_int("BN_CL_GRID_NARROW_BWD_MAX_KB_F32", 16384);
    if (nl > kGridBwdHeld || bytes > static_cast<uint64_t>(most_kb) * 1024u) return false;
  }
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
