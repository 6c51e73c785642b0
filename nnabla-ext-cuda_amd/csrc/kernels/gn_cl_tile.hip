// Channel-last GroupNormalization for groups that are no whole number of
// 16-byte vectors (10, 20, 30, 40, 60 channels: [N,H,W,320] ... [N,H,W,1920] in
// 32 groups), in one pass over x per direction.
//
// x is [N][P][C].  The split kernels (gn_cl_split.cuh) tile the channels into
// 128-byte lines, which only works when a group is 1, 2, 4 or 8 whole vectors.
// Here a block owns whole ROWS instead: PB consecutive positions of one sample
// with all C channels (whole cache lines: C * sizeof(T) is a multiple of 16 and
// the block's range is contiguous memory).  Thread t owns vector t % cv of a row
// (cv = C / VEC) at positions t / cv + k * rpi (rpi = 1024 / cv positions per
// sweep), so element j of its vectors is always the same channel, and it keeps
// one accumulator per element.  The block adds those per group through LDS in a
// fixed order (positions, then the channels of a group), the `split` blocks of
// a sample exchange (mean, m2) - backward: (sum g*dy*xh, sum g*dy) - per group
// as {value, epoch} words (xchg.cuh), merge all parts in block order and finish
// from registers and LDS.  A partner's part that does not arrive is computed
// from global memory in the partner's arithmetic: every wave reaches the end
// whatever the other blocks do, and the result is the same bit for bit.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"
#include "xchg.cuh"

namespace nblahip {

namespace {

constexpr int kTileMaxG = 64;     // groups
constexpr int kTileMaxSplit = 32; // blocks per sample (a bit each in the mask of missing partners)
constexpr int kTileMaxC = 2560;   // channels (backward: column sums and gamma in LDS)

struct ClTileArgs {
  const void *x;
  const void *dy;
  void *out; // y or dx (dx may be null)
  const float *gamma, *beta;
  float *mean, *var; // [N * G]
  const float *dmean, *dvar;
  float *pairs; // backward: [N * split][C][2]
  unsigned long long *xchg;
  uint32_t epoch;
  int spin;
  uint32_t P, C, G;
  uint32_t cv;     // vectors per position
  FastDiv cvd;     // (the same, for t -> (position, vector))
  FastDiv cpgd;    // channels per group, for channel -> group
  FastDiv gd;      // groups, for exchange word -> block
  FastDiv rpid;    // positions per sweep, for positions -> rows that hold one more
  uint32_t rpi;    // positions per sweep = 1024 / cv
  uint32_t active; // threads that own a vector = rpi * cv
  uint32_t split;  // blocks per sample
  uint32_t PB;     // positions per block
  float eps, inv_R, one;
  int accum_dx;
};

__device__ __forceinline__ uint32_t tile_positions(const ClTileArgs &a, uint32_t s) {
  const uint32_t first = s * a.PB;
  return first >= a.P ? 0u : min(a.PB, a.P - first);
}

// The block's per-element values land in cols as [position of the sweep][column]
// (thread t's vector at t * VEC); everything below adds them in a fixed order:
// the same bits in every run, and in a partner that computes this block's part.
template <int VEC>
__device__ __forceinline__ void tile_put_cols(const float (&v)[VEC], const ClTileArgs &a, bool owner,
                                              float *cols) {
  const uint32_t t = threadIdx.x;
  lds_barrier(); // earlier readers of cols and of what is derived from it are done
  if (t < a.active) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) cols[t * VEC + j] = owner ? v[j] : 0.f;
  }
  lds_barrier();
}

// Sum of column c over the positions of the sweep.
__device__ __forceinline__ float tile_column(const ClTileArgs &a, const float *cols, uint32_t c) {
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  uint32_t r = 0;
  for (; r + 4 <= a.rpi; r += 4) {
    s0 += cols[r * a.C + c];
    s1 += cols[(r + 1) * a.C + c];
    s2 += cols[(r + 2) * a.C + c];
    s3 += cols[(r + 3) * a.C + c];
  }
  for (; r < a.rpi; ++r) s0 += cols[r * a.C + c];
  return (s0 + s1) + (s2 + s3);
}

// Forward: (mean, m2) per group from the threads' per-element (mean, m2) over
// their positions, in one trip through LDS.  A thread per column merges the
// rows of the sweep (row r holds full + (r < rem) positions) into the column's
// mean and m2 and leaves them in row 0 of its column (nobody else reads that
// column); a wave per group merges the group's columns - equal counts, so the
// group's mean is the mean of the columns' means and its m2 the sum of theirs
// plus npos * sum (mean_c - mean)^2 - across its lanes.  Nothing is squared
// before its mean is taken off.  tot: [G][2].  Ends with a barrier.
constexpr int kTileColsPerLane = 2; // columns of a group a lane takes: groups of up to 128 channels

template <int VEC>
__device__ __forceinline__ void tile_group_stats(const float (&mu)[VEC], const float (&m2)[VEC],
                                                 const ClTileArgs &a, uint32_t npos, float *cmu,
                                                 float *cm2, float *tot) {
  const uint32_t t = threadIdx.x;
  lds_barrier(); // earlier readers of cmu / cm2 / tot are done
  if (t < a.active) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      cmu[t * VEC + j] = mu[j]; // (threads without a position: zeros, and their rows count nothing)
      cm2[t * VEC + j] = m2[j];
    }
  }
  lds_barrier();
  const uint32_t full = a.rpid.div(npos), rem = npos - full * a.rpi;
  const float fn = static_cast<float>(npos);
  const float inv_n = 1.0f / fn;
  auto rows = [&](uint32_t r) { return static_cast<float>(full + (r < rem ? 1u : 0u)); };
  for (uint32_t c = t; c < a.C; c += kOnchipBlock) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint32_t r = 0;
    for (; r + 4 <= a.rpi; r += 4) {
      s0 = fmaf(rows(r), cmu[r * a.C + c], s0);
      s1 = fmaf(rows(r + 1), cmu[(r + 1) * a.C + c], s1);
      s2 = fmaf(rows(r + 2), cmu[(r + 2) * a.C + c], s2);
      s3 = fmaf(rows(r + 3), cmu[(r + 3) * a.C + c], s3);
    }
    for (; r < a.rpi; ++r) s0 = fmaf(rows(r), cmu[r * a.C + c], s0);
    const float mc = ((s0 + s1) + (s2 + s3)) * inv_n;
    float q0 = 0.f, q1 = 0.f, q2 = 0.f, q3 = 0.f;
    for (r = 0; r + 4 <= a.rpi; r += 4) {
      const float e0 = cmu[r * a.C + c] - mc, e1 = cmu[(r + 1) * a.C + c] - mc;
      const float e2 = cmu[(r + 2) * a.C + c] - mc, e3 = cmu[(r + 3) * a.C + c] - mc;
      q0 = fmaf(rows(r) * e0, e0, q0 + cm2[r * a.C + c]);
      q1 = fmaf(rows(r + 1) * e1, e1, q1 + cm2[(r + 1) * a.C + c]);
      q2 = fmaf(rows(r + 2) * e2, e2, q2 + cm2[(r + 2) * a.C + c]);
      q3 = fmaf(rows(r + 3) * e3, e3, q3 + cm2[(r + 3) * a.C + c]);
    }
    for (; r < a.rpi; ++r) {
      const float e0 = cmu[r * a.C + c] - mc;
      q0 = fmaf(rows(r) * e0, e0, q0 + cm2[r * a.C + c]);
    }
    cmu[c] = mc;
    cm2[c] = (q0 + q1) + (q2 + q3);
  }
  lds_barrier();
  const uint32_t wave = t / kWave, lane = t % kWave;
  const uint32_t cpg = a.cpgd.d;
  const float inv_cpg = 1.0f / static_cast<float>(cpg);
  for (uint32_t g = wave; g < a.G; g += kOnchipBlock / kWave) {
    float cmean[kTileColsPerLane], cq[kTileColsPerLane];
    float lane_means = 0.f;
#pragma unroll
    for (int q = 0; q < kTileColsPerLane; ++q) {
      const uint32_t i = lane + q * kWave;
      const bool has = i < cpg;
      cmean[q] = has ? cmu[g * cpg + i] : 0.f;
      cq[q] = has ? cm2[g * cpg + i] : 0.f;
      lane_means += cmean[q];
    }
    const float mean_g = wave_sum(lane_means) * inv_cpg;
    float lane_q = 0.f;
#pragma unroll
    for (int q = 0; q < kTileColsPerLane; ++q) {
      if (lane + q * kWave < cpg) {
        const float e = cmean[q] - mean_g;
        lane_q += fmaf(fn * e, e, cq[q]);
      }
    }
    lane_q = wave_sum(lane_q);
    if (lane == 0) {
      tot[2 * g] = mean_g;
      tot[2 * g + 1] = lane_q;
    }
  }
  lds_barrier();
}

// Backward: the columns' sums are results of their own (the block's share of
// dgamma / dbeta), so they are kept: a thread per column.  Ends with a barrier.
template <int VEC>
__device__ __forceinline__ void tile_column_sums(const float (&v)[VEC], const ClTileArgs &a,
                                                 bool owner, float *cols, float *csum) {
  tile_put_cols<VEC>(v, a, owner, cols);
  for (uint32_t c = threadIdx.x; c < a.C; c += kOnchipBlock) csum[c] = tile_column(a, cols, c);
  lds_barrier();
}

// Polls the partners' pairs into part[split][2 * G]; a block whose words do
// not turn up gets its bit in *missing_mask.
__device__ __forceinline__ void tile_collect(const ClTileArgs &a, const unsigned long long *slots,
                                             uint32_t self, float *part, uint32_t *missing_mask) {
  const uint32_t pairs = a.split * a.G;
  const FastDiv gd = a.gd;
  for (uint32_t i = threadIdx.x; i < pairs; i += kOnchipBlock) {
    const uint32_t sp = gd.div(i);
    if (sp == self) continue;
    float v0 = 0.f, v1 = 0.f;
    if (xchg_poll2(slots + 2 * i, a.epoch, a.spin, &v0, &v1)) {
      part[2 * i] = v0;
      part[2 * i + 1] = v1;
    } else {
      atomicOr(missing_mask, 1u << sp);
    }
  }
}

} // namespace

// Forward.  Block b = n * split + s (a sample's blocks are neighbours in the
// grid: with more blocks than the chip holds at once, a block's partners are
// running or next in line).
template <typename T, int VEC, int NR, int NS>
__global__ void __launch_bounds__(kOnchipBlock)
gn_cl_tile_fwd_kernel(const ClTileArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NL = NR + NS;
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  __shared__ float cmu[kOnchipBlock * VEC], cm2[kOnchipBlock * VEC];
  __shared__ float tot[2 * kTileMaxG];
  __shared__ float part[kTileMaxSplit * 2 * kTileMaxG];
  __shared__ float merged[2 * kTileMaxG]; // (mean, 1 / std) per group
  __shared__ float gch[kTileMaxC], bch[kTileMaxC];
  __shared__ uint32_t missing_mask;
  const uint32_t t = threadIdx.x;
  const uint32_t n = blockIdx.x / a.split, s = blockIdx.x % a.split;
  uint32_t r = a.cvd.div(t);
  const bool in_sweep = t < a.active;
  const uint32_t tt = in_sweep ? t : 0u;
  r = in_sweep ? r : 0u;
  const uint32_t v = tt - r * a.cv;
  const uint32_t ch = v * VEC;
  const size_t sample = static_cast<size_t>(n) * a.P * a.C;
  const T *__restrict__ x = static_cast<const T *>(a.x) + sample;
  T *__restrict__ y = static_cast<T *>(a.out) + sample;
  unsigned long long *slots = a.xchg + static_cast<size_t>(n) * a.split * 2 * a.G;
  if (t == 0) missing_mask = 0u; // (barriers follow before anyone sets a bit)
  // gamma and beta ahead of the tensor's loads (they travel together), a column
  // per thread; they wait in LDS until the end
  constexpr int kCols = (kTileMaxC + kOnchipBlock - 1) / kOnchipBlock;
  float g_c[kCols], b_c[kCols];
#pragma unroll
  for (int q = 0; q < kCols; ++q) {
    const uint32_t c = t + q * kOnchipBlock;
    g_c[q] = (c < a.C && a.gamma) ? a.gamma[c] : 1.f;
    b_c[q] = (c < a.C && a.beta) ? a.beta[c] : 0.f;
  }
  const uint32_t nb = tile_positions(a, s);
  // (slot k holds a vector: the thread's position against a scalar)
  const int rv = in_sweep ? static_cast<int>(r) : 0x3fffffff;
  auto holds = [&](int k) { return rv < static_cast<int>(nb) - k * static_cast<int>(a.rpi); };
  const size_t base = (static_cast<size_t>(s) * a.PB + r) * a.C + ch;
  const size_t step = static_cast<size_t>(a.rpi) * a.C;

  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k)
      parked[k] = load_raw<T, VEC>(x + (holds(NR + k) ? base + (NR + k) * step : static_cast<size_t>(s) * a.PB * a.C));
#pragma unroll
    for (int k = 0; k < NR; ++k)
      raw[k] = load_raw<T, VEC>(x + (holds(k) ? base + k * step : static_cast<size_t>(s) * a.PB * a.C));
#pragma unroll
    for (int k = 0; k < NS; ++k) spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
#pragma unroll
  for (int q = 0; q < kCols; ++q) {
    const uint32_t c = t + q * kOnchipBlock;
    if (c < a.C) { // (read behind the barriers of the sums)
      gch[c] = g_c[q];
      bch[c] = b_c[q];
    }
  }
  auto slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * kOnchipBlock + t]);
  };

  // (mean, m2) per group of the positions of block sp, from the vectors get(k)
  // (asked for only where slot k lies inside the block); leaves them in tot /
  // returns them to the threads g < G.  Per thread and element a running
  // (mean, m2) over its positions (Welford; the counts' reciprocals are the
  // same correctly rounded floats whether k is a constant or not), then per
  // group mean = sum n*mean_t / count and m2 = sum (m2_t + n*(mean_t - mean)^2).
  auto block_part = [&](uint32_t sp, auto get, auto unrolled, float &pm, float &pq) {
    const uint32_t npos = tile_positions(a, sp);
    const int nk = (in_sweep && r < npos) ? static_cast<int>((npos - 1u - r) / a.rpi + 1u) : 0;
    float mu_t[VEC], m2[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) mu_t[j] = m2[j] = 0.f;
    auto take = [&](int k) {
      const RawVec<T, VEC> x_k = get(k);
      const float rk = 1.0f / static_cast<float>(k + 1);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = elem_fma<T, VEC>(x_k, j, a.one, -mu_t[j]);
        mu_t[j] = fmaf(d, rk, mu_t[j]);
        m2[j] = fmaf(d, elem_fma<T, VEC>(x_k, j, a.one, -mu_t[j]), m2[j]);
      }
    };
    if constexpr (decltype(unrolled)::value) {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        if (k < nk) take(k);
      }
    } else {
#pragma unroll 1
      for (int k = 0; k < nk; ++k) take(k);
    }
    tile_group_stats<VEC>(mu_t, m2, a, npos, cmu, cm2, tot);
    pm = t < a.G ? tot[2 * t] : 0.f;
    pq = t < a.G ? tot[2 * t + 1] : 0.f;
  };

  // ---- this block's part, published; the partners' parts
  float pm, pq;
  block_part(s, [&](int k) { return slot(k); }, std::true_type{}, pm, pq);
  if (t < a.G) {
    part[(s * a.G + t) * 2] = pm;
    part[(s * a.G + t) * 2 + 1] = pq;
    xchg_publish(slots + (s * a.G + t) * 2, pm, a.epoch);
    xchg_publish(slots + (s * a.G + t) * 2 + 1, pq, a.epoch);
  }
  tile_collect(a, slots, s, part, &missing_mask);
  lds_barrier();
  for (uint32_t todo = missing_mask; todo != 0u; todo &= todo - 1u) { // the same in every thread
    const uint32_t sp = static_cast<uint32_t>(__builtin_ctz(todo));
    const size_t pbase = (static_cast<size_t>(sp) * a.PB + r) * a.C + ch;
    block_part(sp, [&](int k) { return load_raw<T, VEC>(x + pbase + k * step); }, std::false_type{}, pm, pq);
    if (t < a.G) {
      part[(sp * a.G + t) * 2] = pm;
      part[(sp * a.G + t) * 2 + 1] = pq;
    }
    lds_barrier();
  }

  // ---- merge in block order (Chan; a thread per group), the statistics
  if (t < a.G) {
    const float cpg = static_cast<float>(a.cpgd.d);
    float m = 0.f, m2 = 0.f, cnt = 0.f;
    for_pairs_in_order(part + t * 2, 2 * static_cast<int>(a.G), static_cast<int>(a.split),
                       [&](int sp, float mb, float qb) {
      const float nbp = static_cast<float>(tile_positions(a, static_cast<uint32_t>(sp))) * cpg;
      if (sp == 0) {
        m = mb;
        m2 = qb;
        cnt = nbp;
        return;
      }
      const float total = cnt + nbp;
      const float d = mb - m;
      const float wgt = nbp / total;
      m = fmaf(d, wgt, m);
      m2 = m2 + qb + d * d * (cnt * wgt);
      cnt = total;
    });
    const float var = m2 * a.inv_R;
    merged[2 * t] = m;
    merged[2 * t + 1] = inv_std(var, a.eps);
    if (s == 0) {
      a.mean[static_cast<size_t>(n) * a.G + t] = m;
      a.var[static_cast<size_t>(n) * a.G + t] = var;
    }
  }
  lds_barrier();

  // ---- normalize what the block holds
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  float sc[VEC], sh[VEC], mu[VEC], bt[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t g = a.cpgd.div(ch + j);
    bt[j] = bch[ch + j];
    mu[j] = merged[2 * g];
    sc[j] = gch[ch + j] * merged[2 * g + 1];
    sh[j] = fmaf(-mu[j], sc[j], bch[ch + j]);
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
          o[j] = fmaf(elem_fma<T, VEC>(x_k, j, a.one, -mu[j]), sc[j], bt[j]);
        }
      }
      store_vec<T, VEC>(y + base + k * step, o);
    }
  }
}

// Backward.  x stays in registers; of dy the first ND vectors of a thread wait
// in LDS, the rest is read a second time for dx (out of L2 for the most part).
// Per column the block's (sum dy*xh, sum dy) is its share of dgamma / dbeta
// (a.pairs, summed over the blocks afterwards); weighted with gamma and added
// over a group's columns they are what the blocks of a sample exchange.
template <typename T, int VEC, int NL, int ND>
__global__ void __launch_bounds__(kOnchipBlock)
gn_cl_tile_bwd_kernel(const ClTileArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  constexpr int NP = ND < NL ? ND : NL;
  __shared__ uint4 park[NP * kOnchipBlock];
  __shared__ float cols[kOnchipBlock * VEC];
  __shared__ float csum[2][kTileMaxC];
  __shared__ float gch[kTileMaxC];
  __shared__ float tot[2][kTileMaxG];
  __shared__ float part[kTileMaxSplit * 2 * kTileMaxG];
  __shared__ float coef[2 * kTileMaxG]; // (cA, cb) per group
  __shared__ uint32_t missing_mask;
  const uint32_t t = threadIdx.x;
  const uint32_t n = blockIdx.x / a.split, s = blockIdx.x % a.split;
  uint32_t r = a.cvd.div(t);
  const bool in_sweep = t < a.active;
  const uint32_t tt = in_sweep ? t : 0u;
  r = in_sweep ? r : 0u;
  const uint32_t v = tt - r * a.cv;
  const uint32_t ch = v * VEC;
  const size_t sample = static_cast<size_t>(n) * a.P * a.C;
  const T *__restrict__ x = static_cast<const T *>(a.x) + sample;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + sample;
  T *__restrict__ dx = a.out ? static_cast<T *>(a.out) + sample : nullptr;
  unsigned long long *slots = a.xchg + static_cast<size_t>(n) * a.split * 2 * a.G;
  if (t == 0) missing_mask = 0u; // (barriers follow before anyone sets a bit)

  // Small loads first, so that they travel with the tensor's: the statistics of
  // each element's group, gamma of the columns, what the thread of group t needs.
  float mean[VEC], istd[VEC], nmi[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const size_t g = static_cast<size_t>(n) * a.G + a.cpgd.div(ch + j);
    mean[j] = a.mean[g];
    istd[j] = a.var[g];
  }
  float g_c[(kTileMaxC + kOnchipBlock - 1) / kOnchipBlock];
#pragma unroll
  for (int q = 0; q < (kTileMaxC + kOnchipBlock - 1) / kOnchipBlock; ++q) {
    const uint32_t c = t + q * kOnchipBlock;
    g_c[q] = (c < a.C && a.gamma) ? a.gamma[c] : 1.f;
  }
  float u_var = 1.f, u_dvar = 0.f, u_dmean = 0.f;
  if (t < a.G) {
    u_var = a.var[static_cast<size_t>(n) * a.G + t];
    if (a.dvar) u_dvar = a.dvar[static_cast<size_t>(n) * a.G + t];
    if (a.dmean) u_dmean = a.dmean[static_cast<size_t>(n) * a.G + t];
  }

  const uint32_t nb = tile_positions(a, s);
  const int rv = in_sweep ? static_cast<int>(r) : 0x3fffffff;
  auto holds = [&](int k) { return rv < static_cast<int>(nb) - k * static_cast<int>(a.rpi); };
  const size_t base = (static_cast<size_t>(s) * a.PB + r) * a.C + ch;
  const size_t step = static_cast<size_t>(a.rpi) * a.C;
  const size_t home = static_cast<size_t>(s) * a.PB * a.C; // a valid address for slots beyond the block
  auto at = [&](int k) { return holds(k) ? base + k * step : home; };

  RawVec<T, VEC> xr[NL];
  {
    RawVec<T, VEC> dr[NP];
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      xr[k] = load_raw<T, VEC>(x + at(k));
      dr[k] = load_raw<T, VEC>(dy + at(k));
    }
#pragma unroll
    for (int k = NP; k < NL; ++k) xr[k] = load_raw<T, VEC>(x + at(k));
#pragma unroll
    for (int k = 0; k < NP; ++k) park[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, dr[k]);
  }
#pragma unroll
  for (int q = 0; q < (kTileMaxC + kOnchipBlock - 1) / kOnchipBlock; ++q) {
    const uint32_t c = t + q * kOnchipBlock;
    if (c < a.C) gch[c] = g_c[q]; // (read behind the barriers of the column sums)
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    istd[j] = inv_std(istd[j], a.eps);
    nmi[j] = -mean[j] * istd[j];
  }
  auto dy_slot = [&](int k) -> RawVec<T, VEC> {
    if (k < NP) return __builtin_bit_cast(RawVec<T, VEC>, park[(k < NP ? k : 0) * kOnchipBlock + t]);
    return load_raw<T, VEC>(dy + at(k));
  };

  // (sum g*dy*xh, sum g*dy) per group of the positions of block sp, from the
  // vectors getx(k), getd(k) (asked for only where slot k lies inside the
  // block), to the threads g < G; the columns' sums stay in csum.
  auto block_sums = [&](uint32_t sp, auto getx, auto getd, auto unrolled, float &p0, float &p1) {
    const uint32_t npos = tile_positions(a, sp);
    const int nk = (in_sweep && r < npos) ? static_cast<int>((npos - 1u - r) / a.rpi + 1u) : 0;
    float sdx[VEC], sdy[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
    auto take = [&](int k) {
      const RawVec<T, VEC> x_k = getx(k);
      const RawVec<T, VEC> d_k = getd(k);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(x_k, j, mean[j], istd[j], nmi[j]);
        sdx[j] = elem_fma<T, VEC>(d_k, j, xh, sdx[j]);
        sdy[j] = elem_fma<T, VEC>(d_k, j, a.one, sdy[j]);
      }
    };
    if constexpr (decltype(unrolled)::value) {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        if (k < nk) take(k);
      }
    } else {
#pragma unroll 1
      for (int k = 0; k < nk; ++k) take(k);
    }
    tile_column_sums<VEC>(sdx, a, nk > 0, cols, csum[0]);
    tile_column_sums<VEC>(sdy, a, nk > 0, cols, csum[1]);
    const uint32_t wave = t / kWave, lane = t % kWave;
    const uint32_t cpg = a.cpgd.d;
    for (uint32_t g = wave; g < a.G; g += kOnchipBlock / kWave) {
      float s0 = 0.f, s1 = 0.f;
      for (uint32_t i = lane; i < cpg; i += kWave) {
        const float w = gch[g * cpg + i];
        s0 = fmaf(w, csum[0][g * cpg + i], s0);
        s1 = fmaf(w, csum[1][g * cpg + i], s1);
      }
      s0 = wave_sum(s0);
      s1 = wave_sum(s1);
      if (lane == 0) {
        tot[0][g] = s0;
        tot[1][g] = s1;
      }
    }
    lds_barrier();
    p0 = t < a.G ? tot[0][t] : 0.f;
    p1 = t < a.G ? tot[1][t] : 0.f;
  };

  // ---- this block's part: the columns' pairs to memory, the groups' published
  float p0, p1;
  block_sums(s, [&](int k) { return xr[k]; }, dy_slot, std::true_type{}, p0, p1);
  if (a.pairs) {
    float2 *out = reinterpret_cast<float2 *>(a.pairs) + (static_cast<size_t>(n) * a.split + s) * a.C;
    for (uint32_t c = t; c < a.C; c += kOnchipBlock) out[c] = make_float2(csum[0][c], csum[1][c]);
  }
  if (t < a.G) {
    part[(s * a.G + t) * 2] = p0;
    part[(s * a.G + t) * 2 + 1] = p1;
    xchg_publish(slots + (s * a.G + t) * 2, p0, a.epoch);
    xchg_publish(slots + (s * a.G + t) * 2 + 1, p1, a.epoch);
  }
  if (dx == nullptr) return;

  // ---- the partners' parts
  tile_collect(a, slots, s, part, &missing_mask);
  lds_barrier();
  for (uint32_t todo = missing_mask; todo != 0u; todo &= todo - 1u) { // the same in every thread
    const uint32_t sp = static_cast<uint32_t>(__builtin_ctz(todo));
    const size_t pbase = (static_cast<size_t>(sp) * a.PB + r) * a.C + ch;
    block_sums(sp, [&](int k) { return load_raw<T, VEC>(x + pbase + k * step); },
               [&](int k) { return load_raw<T, VEC>(dy + pbase + k * step); }, std::false_type{}, p0, p1);
    if (t < a.G) {
      part[(sp * a.G + t) * 2] = p0;
      part[(sp * a.G + t) * 2 + 1] = p1;
    }
    lds_barrier();
  }

  // ---- totals in block order and the group's coefficients (a thread per group)
  if (t < a.G) {
    float t2 = 0.f, s1 = 0.f;
    for_pairs_in_order(part + t * 2, 2 * static_cast<int>(a.G), static_cast<int>(a.split),
                       [&](int, float q0, float q1) {
      t2 += q0;
      s1 += q1;
    });
    const float vpe = u_var + a.eps;
    const float is = 1.0f / sqrtf(vpe);
    coef[2 * t] = -is * t2 * a.inv_R + (a.dvar ? 2.f * u_dvar * (vpe * is) * a.inv_R : 0.f);
    coef[2 * t + 1] = -s1 * is * a.inv_R + (a.dmean ? u_dmean * a.inv_R : 0.f);
  }
  lds_barrier();

  // ---- dx.  half: dx = dy*gis + x*A2 + B2 with A2 = istd*cA, B2 = nmi*cA + cb
  // (two mixed-precision fmas per element); float: dx = dy*gis + xh*cA + cb
#pragma unroll
  for (int k = 0; k < NL; ++k) forget<T, VEC>(xr[k]);
  float gis[VEC], cA[VEC], cb[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t g = a.cpgd.div(ch + j);
    const float ca = coef[2 * g], cbu = coef[2 * g + 1];
    gis[j] = gch[ch + j] * istd[j];
    if constexpr (sizeof(T) == 2) {
      cA[j] = istd[j] * ca;
      cb[j] = fmaf(nmi[j], ca, cbu);
    } else {
      cA[j] = ca;
      cb[j] = cbu;
    }
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    if (holds(k)) {
      const RawVec<T, VEC> d_k = dy_slot(k);
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(d_k, j, gis[j], elem_fma<T, VEC>(xr[k], j, cA[j], cb[j]));
        } else {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean[j], istd[j], nmi[j]);
          o[j] = elem_fma<T, VEC>(d_k, j, gis[j], fmaf(xh, cA[j], cb[j]));
        }
      }
      T *q = dx + base + k * step;
      if (a.accum_dx) {
        float old[VEC];
        load_vec<T, VEC>(q, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] += old[j];
      }
      store_vec<T, VEC>(q, o);
    }
  }
}

namespace {

struct TilePlan {
  bool ok = false;
  int nl = 0;
  uint32_t cv = 0, rpi = 0, split = 0, pb = 0;
};

// Blocks per sample: enough for a block per CU, more where a block's share
// would not fit `max_nl` vectors per thread.
TilePlan plan_tile(const ClProblem &p, bool aligned, int max_nl) {
  TilePlan pl;
  if (!aligned || !tune_int("GN_CL_TILE", 1)) return pl;
  if (!p.bc_gamma || !p.bc_beta || p.groups == p.channels) return pl;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.channels % vec != 0 || p.channels > kTileMaxC || p.groups > kTileMaxG) return pl;
  // A block whose partner's word does not arrive reads the partner's positions
  // of x (and dy) again, which the partner may already be overwriting in place.
  const uint64_t tensor_bytes = static_cast<uint64_t>(p.batch * p.spatial * p.channels) * (16 / vec);
  if (ranges_overlap(p.out, p.x, tensor_bytes) || ranges_overlap(p.out, p.dy, tensor_bytes)) return pl;
  if (p.channels % p.groups != 0 || p.channels / p.groups > kTileColsPerLane * kWave) return pl;
  const int64_t cv = p.channels / vec;
  if (cv > 512) return pl;
  const int64_t rpi = kOnchipBlock / cv;
  const int64_t cus = device_cus();
  int64_t split = std::min<int64_t>(kTileMaxSplit, std::max<int64_t>(1, (cus + p.batch - 1) / p.batch));
  split = std::min<int64_t>(split, (p.spatial + rpi - 1) / rpi);
  auto nl_of = [&](int64_t s) {
    const int64_t pb = (p.spatial + s - 1) / s;
    return (pb + rpi - 1) / rpi;
  };
  while (nl_of(split) > max_nl && split < kTileMaxSplit) ++split;
  if (split > kTileMaxSplit || nl_of(split) > max_nl) return pl;
  const int64_t pb = (p.spatial + split - 1) / split;
  split = (p.spatial + pb - 1) / pb; // every block holds a position
  if (p.batch * split * 100 < cus * tune_int("GN_CL_TILE_MIN_PCT", 1)) return pl;
  // Partners wait for each other: a block per CU at most, all there at once.
  if (p.batch * split > cus) return pl;
  if (static_cast<size_t>(p.batch) * split * 2 * p.groups > xchg_capacity()) return pl;
  pl.ok = true;
  pl.nl = static_cast<int>(nl_of(split));
  pl.cv = static_cast<uint32_t>(cv);
  pl.rpi = static_cast<uint32_t>(rpi);
  pl.split = static_cast<uint32_t>(split);
  pl.pb = static_cast<uint32_t>(pb);
  return pl;
}

ClTileArgs tile_args(const ClProblem &p, const TilePlan &pl) {
  ClTileArgs a{};
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.spin = tune_int("XCHG_SPIN", 64);
  a.P = static_cast<uint32_t>(p.spatial);
  a.C = static_cast<uint32_t>(p.channels);
  a.G = static_cast<uint32_t>(p.groups);
  a.cv = pl.cv;
  a.cvd = FastDiv(pl.cv);
  a.cpgd = FastDiv(static_cast<uint32_t>(p.channels / p.groups));
  a.gd = FastDiv(static_cast<uint32_t>(p.groups));
  a.rpid = FastDiv(pl.rpi);
  a.rpi = pl.rpi;
  a.active = pl.rpi * pl.cv;
  a.split = pl.split;
  a.PB = pl.pb;
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * (p.channels / p.groups)));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  return a;
}

// Vectors per thread the forward holds: 13 (half: the per-element scale and
// shift take 16 registers more than float's) or 16 in registers, 3 (half: its
// per-element statistics take 64 KB of LDS on their way to the groups) or 5 in LDS.
constexpr int tile_fwd_max(int dtype) { return dtype == NBLAHIP_F16 ? 16 : 21; }

template <typename T, int VEC>
int run_tile_fwd(int nl, const ClTileArgs &a, unsigned grid, hipStream_t st) {
  constexpr int kTop = sizeof(T) == 2 ? 13 : 16;
#define TILE_CASE(NR, NS)                                                                        \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH("gn_cl_tile_fwd_kernel", (gn_cl_tile_fwd_kernel<T, VEC, NR, NS>), dim3(grid), \
                   dim3(kOnchipBlock), 0, st, a);                                                \
    return last_launch_status();                                                                 \
  }
  TILE_CASE(3, 0)
  TILE_CASE(6, 0)
  TILE_CASE(9, 0)
  if constexpr (sizeof(T) == 4) {
    TILE_CASE(12, 0)
  } else {
    TILE_CASE(11, 0)
  }
  TILE_CASE(kTop, 0)
  TILE_CASE(kTop, 2)
  if constexpr (sizeof(T) == 2) {
    TILE_CASE(kTop, 3)
  } else {
    TILE_CASE(kTop, 5)
  }
#undef TILE_CASE
  return NBLAHIP_EINVAL;
}

// Vectors per thread the backward holds of x (registers); dy beyond ND vectors
// is read twice.
constexpr int tile_bwd_max(int dtype) { return dtype == NBLAHIP_F16 ? 12 : 16; }

template <typename T, int VEC>
int run_tile_bwd(int nl, const ClTileArgs &a, unsigned grid, hipStream_t st) {
  constexpr int ND = sizeof(T) == 2 ? 5 : 6;
#define TILE_CASE(NL)                                                                            \
  if (nl <= (NL)) {                                                                              \
    NBLAHIP_LAUNCH("gn_cl_tile_bwd_kernel", (gn_cl_tile_bwd_kernel<T, VEC, NL, ND>), dim3(grid), \
                   dim3(kOnchipBlock), 0, st, a);                                                \
    return last_launch_status();                                                                 \
  }
  TILE_CASE(2)
  TILE_CASE(4)
  TILE_CASE(6)
  TILE_CASE(9)
  TILE_CASE(12)
  if constexpr (sizeof(T) == 4) {
    TILE_CASE(16)
  }
#undef TILE_CASE
  return NBLAHIP_EINVAL;
}

} // namespace

bool cl_tile_bwd(const ClProblem &p, bool aligned, float **pairs, int64_t *pair_batches,
                 hipStream_t st, int *status) {
  const TilePlan pl = plan_tile(p, aligned, tile_bwd_max(p.dtype));
  if (!pl.ok) return false;
  ClTileArgs a = tile_args(p, pl);
  if (!xchg_acquire(static_cast<size_t>(p.batch) * pl.split * 2 * p.groups, st, &a.xchg, &a.epoch, status))
    return *status != 0;
  a.pairs = static_cast<float *>(p.ws); // [batch * split][C][2], summed over its first axis afterwards
  *pairs = a.pairs;
  *pair_batches = p.batch * pl.split;
  const unsigned grid = static_cast<unsigned>(p.batch * pl.split);
  *status = p.dtype == NBLAHIP_F16 ? run_tile_bwd<__half, 8>(pl.nl, a, grid, st)
                                   : run_tile_bwd<float, 4>(pl.nl, a, grid, st);
  return true;
}

bool cl_tile_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status) {
  const TilePlan pl = plan_tile(p, aligned, tile_fwd_max(p.dtype));
  if (!pl.ok) return false;
  ClTileArgs a = tile_args(p, pl);
  if (!xchg_acquire(static_cast<size_t>(p.batch) * pl.split * 2 * p.groups, st, &a.xchg, &a.epoch, status))
    return *status != 0;
  const unsigned grid = static_cast<unsigned>(p.batch * pl.split);
  *status = p.dtype == NBLAHIP_F16 ? run_tile_fwd<__half, 8>(pl.nl, a, grid, st)
                                   : run_tile_fwd<float, 4>(pl.nl, a, grid, st);
  return true;
}

} // namespace nblahip
