// Channel-last Group/InstanceNormalization with a reduction unit SPLIT over
// several workgroups that exchange their partial sums.
//
// x is [N][P][C].  A statistics unit (a group of a sample, or one channel of a
// sample) is a strided tile of P positions x a few channels, i.e. a 2- to
// 128-byte piece of every 128-byte cache line it touches.  A block that owns
// whole units therefore reads pieces of lines (gn_cl_rows.cuh), and the other
// pieces are fetched again by the blocks that own the neighbouring units.
//
// Here a block owns whole LINES instead: a column tile of 8 sixteen-byte
// vectors (128 bytes: 64 half or 32 float channels, all the units inside it)
// over PB consecutive positions.  The `split` blocks that cover the P positions
// of one (sample, column tile) each reduce their part in registers, publish the
// partial sums of every unit in the tile, read the partials of their partner
// blocks, merge all of them in the same fixed order (every block arrives at
// bit-identical statistics) and finish their part from registers: one pass
// over HBM per direction, in whole lines, with many small blocks per CU.
//
// The partials travel as {value, epoch} words (xchg.cuh): no barrier, no fence,
// no zeroed memory.  A block polls each word at most `spin` times; if a partner
// has not published by then, the block computes that partner's partial itself
// from global memory, in the partner's own arithmetic: every wave reaches the
// end of the kernel whatever the other blocks do, and the result is the same
// bit for bit either way.
#pragma once

#include "common.cuh"
#include "launch.hpp"
#include "xchg.cuh"

namespace nblahip {

constexpr int kSplitTV = 8;    // 16-byte vectors per column tile (one 128-byte line per position)
constexpr int kSplitMax = kClSplitMaxBlocks; // most blocks per (sample, column tile)

struct ClSplitArgs {
  const void *x;
  const void *dy; // backward
  void *out;      // y or dx (dx may be null)
  const float *gamma;
  const float *beta;
  float *mean; // forward: written, backward: read; [N * C / cpg]
  float *var;
  const float *dmean;
  const float *dvar;
  float *pairs;             // backward: [N * split][C][2] = (sum dy*xh, sum dy) per block and channel
  unsigned long long *xchg; // this call's exchange words
  uint32_t epoch;
  int spin;  // polls per exchange word before the partner's part is recomputed
  int P, C;
  int tiles; // column tiles per position = C * sizeof(T) / 128
  int split; // blocks per (sample, column tile)
  int PB;    // positions per block = NL * TPR / 8
  int cpg;   // channels per unit (1: instances)
  int cvg_shift; // log2 of the vectors per unit (groups only)
  float eps, inv_R, one;
  int accum_dx;
  // Block order: 0: the column tile runs fastest (b = (n * split + s) * tiles +
  // tile), 1: the blocks of a (sample, tile) are neighbours (b = (n * tiles +
  // tile) * split + s) - for grids beyond what the chip holds at once, where a
  // block's partners must not be a whole round of blocks away.
  int partners_adjacent;
  // BatchNormalization through these kernels (one sample, a unit per channel):
  // running statistics to update, may be null.
  float *rmean, *rvar;
  float decay, unbias;
};

// (column tile, block of the plane, sample) of block b.
__device__ __forceinline__ void split_block_coords(const ClSplitArgs &a, uint32_t b, uint32_t &tile,
                                                   uint32_t &s, uint32_t &n) {
  if (a.partners_adjacent) {
    s = b % a.split;
    const uint32_t nt = b / a.split;
    tile = nt % a.tiles;
    n = nt / a.tiles;
  } else {
    tile = b % a.tiles;
    const uint32_t ns = b / a.tiles;
    s = ns % a.split;
    n = ns / a.split;
  }
}

// Polls the partners' words into part[] (a thread takes the two words of a
// unit at a time, the first reads of up to four units in flight together: a
// tile of an instance in 16 blocks of 256 threads has 1920 words to collect per
// block, four round trips one after the other when polled unit by unit); words
// that do not turn up mark their block in missing[] (and missing[kSplitMax]:
// "any at all", the one flag a block reads when every word has arrived).
template <int TPR>
__device__ __forceinline__ void split_collect(const ClSplitArgs &a, const unsigned long long *base,
                                              uint32_t self, int per, float *part, int *missing) {
  constexpr int kFly = TPR >= 1024 ? 1 : (TPR >= 512 ? 2 : 4); // 2048 words a sweep
  const int total = a.split * per;
  for (int i0 = 2 * threadIdx.x; i0 < total; i0 += 2 * TPR * kFly) {
    unsigned long long w[kFly][2];
    bool want[kFly];
#pragma unroll
    for (int f = 0; f < kFly; ++f) {
      const int idx = i0 + f * 2 * TPR;
      want[f] = idx < total && idx / per != static_cast<int>(self);
      if (want[f]) {
        w[f][0] = __hip_atomic_load(base + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w[f][1] = __hip_atomic_load(base + idx + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
#pragma unroll
    for (int f = 0; f < kFly; ++f) {
      if (!want[f]) continue;
      const int idx = i0 + f * 2 * TPR;
      float v0, v1;
      bool ok = a.spin > 0 && static_cast<uint32_t>(w[f][0] >> 32) == a.epoch &&
                static_cast<uint32_t>(w[f][1] >> 32) == a.epoch;
      if (ok) {
        v0 = __uint_as_float(static_cast<uint32_t>(w[f][0]));
        v1 = __uint_as_float(static_cast<uint32_t>(w[f][1]));
      } else {
        ok = xchg_poll2(base + idx, a.epoch, a.spin - 1, &v0, &v1);
      }
      if (ok) {
        part[idx] = v0;
        part[idx + 1] = v1;
      } else {
        missing[idx / per] = 1;
        missing[kSplitMax] = 1;
      }
    }
  }
}

// Publishes this block's entries of part[] (a word per thread).
template <int TPR>
__device__ __forceinline__ void split_publish_own(const ClSplitArgs &a, unsigned long long *base,
                                                  uint32_t self, int per, const float *part) {
  lds_barrier(); // part[self] as its writers left it
  for (int e = threadIdx.x; e < per; e += TPR)
    xchg_publish(base + self * per + e, part[self * per + e], a.epoch);
}

// Sum of v over the threads of the block that hold the same unit of the tile
// (groups: the 2^cvg_shift neighbouring vectors of a position; every thread of
// a unit receives the total).  fold: [TPR / 64][8].
template <int TPR>
__device__ __forceinline__ float split_group_sum(float v, int cvg_shift, uint32_t cvx, uint32_t gi,
                                                 float (*fold)[kSplitTV]) {
  constexpr int NW = TPR / kWave;
  v = lanes_sum_below(v, 1u << cvg_shift);
  v = lanes_sum_from(v, 8u);
  lds_barrier(); // earlier readers of fold are done
  if ((threadIdx.x & (kWave - 1)) < kSplitTV && (cvx & ((1u << cvg_shift) - 1)) == 0)
    fold[threadIdx.x / kWave][gi] = v;
  lds_barrier();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) t += fold[w][gi];
  return t;
}

// The same for VEC per-channel values of a thread (instances): threads with
// equal cvx hold the same channels.  Butterfly over the lanes 8 apart, a row of
// fold[TPR / 64][8 * VEC] per wave, the rows added in wave order by one thread
// per channel (tot[8 * VEC]); v[j] = total of channel cvx * VEC + j.
template <int TPR, int VEC>
__device__ __forceinline__ void split_channel_sums(float (&v)[VEC], uint32_t cvx,
                                                   float (*fold)[kSplitTV * VEC], float *tot) {
  constexpr int NW = TPR / kWave;
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = xor_add<32>(xor_add<16>(xor_add<8>(v[j])));
  lds_barrier(); // earlier readers of fold / tot are done
  if ((threadIdx.x & (kWave - 1)) < kSplitTV) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fold[threadIdx.x / kWave][cvx * VEC + j] = v[j];
  }
  lds_barrier();
  if (threadIdx.x < kSplitTV * VEC) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w][threadIdx.x];
    tot[threadIdx.x] = t;
  }
  lds_barrier();
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = tot[cvx * VEC + j];
}

// Backward: the per-channel pairs (sum dy*xh, sum dy) of the block, both at
// once, straight into chs[2][8 * VEC] (nothing returns to the threads).
// fold: [TPR / 64][2 * 8 * VEC].
template <int TPR, int VEC>
__device__ __forceinline__ void split_pair_sums(float (&sdx)[VEC], float (&sdy)[VEC], uint32_t cvx,
                                                float (*fold)[2 * kSplitTV * VEC],
                                                float (*chs)[kSplitTV * VEC]) {
  constexpr int NW = TPR / kWave;
  constexpr int CH = kSplitTV * VEC;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    sdx[j] = xor_add<32>(xor_add<16>(xor_add<8>(sdx[j])));
    sdy[j] = xor_add<32>(xor_add<16>(xor_add<8>(sdy[j])));
  }
  lds_barrier(); // earlier readers of fold / chs are done
  if ((threadIdx.x & (kWave - 1)) < kSplitTV) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      fold[threadIdx.x / kWave][cvx * VEC + j] = sdx[j];
      fold[threadIdx.x / kWave][CH + cvx * VEC + j] = sdy[j];
    }
  }
  lds_barrier();
  for (int e = threadIdx.x; e < 2 * CH; e += TPR) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += fold[w][e];
    chs[e / CH][e % CH] = t;
  }
  lds_barrier();
}

__device__ __forceinline__ float split_count(const ClSplitArgs &a, int sp) {
  const int left = a.P - sp * a.PB;
  return static_cast<float>(left < a.PB ? left : a.PB);
}

// Chan merge of the (mean, m2) partials of one unit over the blocks, in block
// order; counts follow from the geometry.  Returns mean, var (biased).
__device__ __forceinline__ void split_merge_stats(const ClSplitArgs &a, const float *part, int per,
                                                  int u, float per_pos, float &mean, float &var) {
  float m = 0.f, m2 = 0.f, n = 0.f;
  for_pairs_in_order(part + u * 2, per, a.split, [&](int sp, float mb, float qb) {
    const float nb = split_count(a, sp) * per_pos;
    if (sp == 0) {
      m = mb;
      m2 = qb;
      n = nb;
      return;
    }
    const float tot = n + nb;
    const float d = mb - m;
    const float wgt = nb / tot;
    m = fmaf(d, wgt, m);
    m2 = m2 + qb + d * d * (n * wgt);
    n = tot;
  });
  mean = m;
  var = m2 * a.inv_R;
}

// The (mean, m2) part of block sp of a sample for the thread's units, from
// sums every wave takes over its OWN vectors as its loads arrive (the memory
// system serves a CU's waves one after the other: what a wave does before the
// block's first barrier hides behind the other waves' loads; a second pass
// about the block's mean kept memory idle).  Per thread and unit: s = sum x,
// then about the thread's own mean K = s / n: s1 = sum (x - K) (rounding
// residue), s2 = sum (x - K)^2; then mean = sum_t s / count and, about it,
// m2 = sum_t (s2 + 2 e s1 + n e^2) with e = K - mean: two block sums of a few
// operations per thread.  sum_t n e^2 is the variance between the threads'
// means, never more than m2 itself: nothing cancels, whatever the data.
// get(k): the vector at position sp * PB + prow + k * PR (asked for only where
// that lies inside the plane).  ROLLED: loops (vectors from global memory, few
// registers) instead of straight-line code; the arithmetic is the same,
// element by element.
template <typename T, int VEC, int NL, int TPR, bool INSTANCE, bool ROLLED, class Get>
__device__ __forceinline__ void split_block_part(const ClSplitArgs &a, int sp, uint32_t prow,
                                                 uint32_t cvx, uint32_t gi, float per_pos, Get get,
                                                 float (*fold)[kSplitTV * (INSTANCE ? VEC : 1)],
                                                 float *tot, float (&m)[INSTANCE ? VEC : 1],
                                                 float (&q)[INSTANCE ? VEC : 1]) {
  constexpr int PR = TPR / kSplitTV;
  constexpr int SV = INSTANCE ? VEC : 1;
  const int left = a.P - sp * a.PB - static_cast<int>(prow); // positions from the thread's first on
  const int nk = left <= 0 ? 0 : min(NL, (left + PR - 1) / PR); // the thread's vectors
  float kk[SV], s1[SV], s2[SV];
#pragma unroll
  for (int j = 0; j < SV; ++j) m[j] = s1[j] = s2[j] = 0.f;
  auto add = [&](int k) {
    const RawVec<T, VEC> r = get(k);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int ju = INSTANCE ? j : 0;
      m[ju] = elem_fma<T, VEC>(r, j, a.one, m[ju]);
    }
  };
  auto take = [&](int k) {
    const RawVec<T, VEC> r = get(k);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int ju = INSTANCE ? j : 0;
      const float d = elem_fma<T, VEC>(r, j, a.one, -kk[ju]);
      s1[ju] += d;
      s2[ju] = fmaf(d, d, s2[ju]);
    }
  };
  const float nt = static_cast<float>(nk * (INSTANCE ? 1 : VEC));
  const float rnt = 1.0f / fmaxf(nt, 1.f);
  if constexpr (ROLLED) {
#pragma unroll 1
    for (int k = 0; k < nk; ++k) add(k);
#pragma unroll
    for (int j = 0; j < SV; ++j) kk[j] = m[j] * rnt;
#pragma unroll 1
    for (int k = 0; k < nk; ++k) take(k);
  } else {
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (k < nk) add(k);
    }
#pragma unroll
    for (int j = 0; j < SV; ++j) kk[j] = m[j] * rnt;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      if (k < nk) take(k);
    }
  }
  const float cnt = split_count(a, sp) * per_pos;
  if constexpr (INSTANCE) {
    split_channel_sums<TPR, VEC>(m, cvx, fold, tot);
    const float icnt = 1.0f / cnt;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      m[j] *= icnt;
      const float e = kk[j] - m[j];
      q[j] = fmaf(e, fmaf(nt, e, 2.f * s1[j]), s2[j]);
    }
    split_channel_sums<TPR, VEC>(q, cvx, fold, tot);
  } else {
    m[0] = split_group_sum<TPR>(m[0], a.cvg_shift, cvx, gi, fold) / cnt;
    const float e = kk[0] - m[0];
    q[0] = split_group_sum<TPR>(fmaf(e, fmaf(nt, e, 2.f * s1[0]), s2[0]), a.cvg_shift, cvx, gi, fold);
  }
}

// ---------------------------------------------------------------------------
// Forward.  Block b = ((n * split + s) * tiles + tile); thread t owns vector
// t % 8 of the tile at positions s * PB + t / 8 + k * (TPR / 8), k < NL.
// ---------------------------------------------------------------------------
// MANY: more than 16 blocks per (sample, column tile); their partials lie in
// LDS sized by the launch (BatchNormalization's single plane of all rows).
template <typename T, int VEC, int NL, int TPR, bool INSTANCE, bool MANY = false>
__global__ void __launch_bounds__(TPR)
cl_split_fwd_kernel(const ClSplitArgs a) {
  constexpr int TV = kSplitTV;
  constexpr int PR = TPR / TV;
  constexpr int NW = TPR / kWave;
  constexpr int UMAX = INSTANCE ? TV * VEC : TV;
  __shared__ float fold[NW][UMAX];
  __shared__ float tot[UMAX];
  __shared__ float part16[MANY ? 1 : 16 * UMAX * 2];
  extern __shared__ float part_many[]; // [split][2 * units of the tile], sized by the launch
  float *const part = MANY ? part_many : part16;
  __shared__ float merged[UMAX * 2]; // (mean, 1 / std) per unit
  __shared__ int missing[kSplitMax + 1];
  uint32_t tile, s, n;
  split_block_coords(a, blockIdx.x, tile, s, n);
  const uint32_t cvx = threadIdx.x % TV, prow = threadIdx.x / TV;
  const uint32_t ch = (tile * TV + cvx) * VEC;
  const uint32_t gi = INSTANCE ? 0u : (cvx >> a.cvg_shift);
  const int U = INSTANCE ? TV * VEC : (TV >> a.cvg_shift); // units in the tile
  const int per = 2 * U;
  const float per_pos = INSTANCE ? 1.f : static_cast<float>(a.cpg);
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(n) * a.P * a.C + ch;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(n) * a.P * a.C + ch;
  unsigned long long *slots =
      a.xchg + (static_cast<size_t>(n) * a.tiles + tile) * a.split * per;
  const bool writer = prow == 0 && (INSTANCE || (cvx & ((1u << a.cvg_shift) - 1)) == 0);

  if (threadIdx.x <= kSplitMax) missing[threadIdx.x] = 0;
  auto unit_index = [&]() -> size_t { // statistics index of unit threadIdx.x of the tile
    return INSTANCE ? static_cast<size_t>(n) * a.C + tile * TV * VEC + threadIdx.x
                    : static_cast<size_t>(n) * (a.C / a.cpg) + (tile * TV * VEC) / a.cpg + threadIdx.x;
  };
  float unit_mean = 0.f, unit_var = 0.f; // kept for the running statistics
  // gamma and beta of the tile's channels: one coalesced load each by the
  // first wave, ahead of the tensor's loads (they travel together), handed on
  // through LDS behind the barriers of the block's part.  (Every thread loading
  // its own VEC channels is 2 * VEC loads per wave in front of the tensor's.)
  __shared__ float gb[2][TV * VEC];
  float g_t = 1.f, b_t = 0.f;
  if (threadIdx.x < TV * VEC) {
    if (a.gamma) g_t = a.gamma[tile * TV * VEC + threadIdx.x];
    if (a.beta) b_t = a.beta[tile * TV * VEC + threadIdx.x];
  }
  RawVec<T, VEC> raw[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = s * a.PB + prow + k * PR;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    raw[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + static_cast<size_t>(ok ? pos : s * a.PB) * a.C));
  }
  if (threadIdx.x < TV * VEC) {
    gb[0][threadIdx.x] = g_t;
    gb[1][threadIdx.x] = b_t;
  }

  float mean[INSTANCE ? VEC : 1], var[INSTANCE ? VEC : 1];
  // ---- this block's part
  split_block_part<T, VEC, NL, TPR, INSTANCE, false>(
      a, static_cast<int>(s), prow, cvx, gi, per_pos, [&](int k) { return raw[k]; }, fold, tot, mean, var);
  if (writer) {
#pragma unroll
    for (int j = 0; j < (INSTANCE ? VEC : 1); ++j) {
      const int u = INSTANCE ? static_cast<int>(cvx) * VEC + j : static_cast<int>(gi);
      part[s * per + u * 2] = mean[j];
      part[s * per + u * 2 + 1] = var[j];
    }
  }

  // ---- the partners' parts
  split_publish_own<TPR>(a, slots, s, per, part);
  split_collect<TPR>(a, slots, s, per, part, missing);
  lds_barrier();
  const bool any_missing = missing[kSplitMax] != 0; // (a flag per partner costs an LDS round trip each)
  for (int sp = 0; any_missing && sp < a.split; ++sp) {
    if (sp == static_cast<int>(s) || !missing[sp]) continue; // same answer in every thread
    // Partner sp has not published: its part from global memory, one vector
    // at a time (the block's own vectors stay in registers).
    split_block_part<T, VEC, NL, TPR, INSTANCE, true>(
        a, sp, prow, cvx, gi, per_pos,
        [&](int k) {
          return load_raw<T, VEC>(x + static_cast<size_t>(sp * a.PB + prow + k * PR) * a.C);
        },
        fold, tot, mean, var);
    if (writer) {
#pragma unroll
      for (int j = 0; j < (INSTANCE ? VEC : 1); ++j) {
        const int u = INSTANCE ? static_cast<int>(cvx) * VEC + j : static_cast<int>(gi);
        part[sp * per + u * 2] = mean[j];
        part[sp * per + u * 2 + 1] = var[j];
      }
    }
    lds_barrier();
  }

  // ---- merge in block order (a thread per unit: every thread merging its own
  // units again cost 2.6 us in a 1024-thread block of an instance), write the
  // statistics (first block), normalize
  if (static_cast<int>(threadIdx.x) < U) {
    const int u = static_cast<int>(threadIdx.x);
    float m, v;
    split_merge_stats(a, part, per, u, per_pos, m, v);
    merged[2 * u] = m;
    merged[2 * u + 1] = inv_std(v, a.eps); // once per unit, not once per thread and channel
    if (s == 0) {
      const size_t ug = unit_index();
      a.mean[ug] = m;
      a.var[ug] = v;
      unit_mean = m;
      unit_var = v;
    }
  }
  lds_barrier();
#pragma unroll
  for (int j = 0; j < (INSTANCE ? VEC : 1); ++j) {
    const int u = INSTANCE ? static_cast<int>(cvx) * VEC + j : static_cast<int>(gi);
    mean[j] = merged[2 * u];
    var[j] = merged[2 * u + 1]; // (1 / std from here on)
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
  float sc[VEC], sh[VEC], mu[VEC], bet[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int ju = INSTANCE ? j : 0;
    bet[j] = gb[1][cvx * VEC + j];
    sc[j] = gb[0][cvx * VEC + j] * var[ju];
    mu[j] = mean[ju];
    sh[j] = fmaf(-mean[ju], sc[j], bet[j]);
  }
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = s * a.PB + prow + k * PR;
    if (pos < static_cast<uint32_t>(a.P)) {
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(raw[k], j, sc[j], sh[j]);
        } else {
          o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mu[j]), sc[j], bet[j]);
        }
      }
      store_vec<T, VEC>(y + static_cast<size_t>(pos) * a.C, o);
    }
  }
  // BatchNormalization: the running statistics, by the unit threads of the
  // plane's first block.  At the very end: their loads cost this wave a round
  // trip that nothing else waits for (ahead of the tensor's loads the test for
  // them cost every Group/InstanceNormalization forward 0.4 us).
  if (a.rmean && s == 0 && static_cast<int>(threadIdx.x) < U) {
    const size_t ug = unit_index();
    a.rmean[ug] = a.decay * a.rmean[ug] + (1.f - a.decay) * unit_mean;
    a.rvar[ug] = a.decay * a.rvar[ug] + (1.f - a.decay) * unit_var * a.unbias;
  }
}

// The per-channel pairs of block (sample of x / dy, sp) from global memory into
// chs, a vector at a time, in the arithmetic of the block that owns them: the
// positions in the order of its registers, the same folds.  x, dy: the
// thread's column of the sample; mean, istd, nmi: the sample's statistics for
// the thread's units.
template <typename T, int VEC, int NL, int TPR, bool INSTANCE, int SV>
__device__ __forceinline__ void split_pairs_from_memory(
    const ClSplitArgs &a, const T *__restrict__ x, const T *__restrict__ dy, int sp, uint32_t prow,
    uint32_t cvx, const float (&mean)[SV], const float (&istd)[SV], const float (&nmi)[SV],
    float (*fold)[2 * kSplitTV * VEC], float (*chs)[kSplitTV * VEC]) {
  constexpr int PR = TPR / kSplitTV;
  float sdx[VEC], sdy[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll 1
  for (int k = 0; k < NL; ++k) {
    const uint32_t pos = sp * a.PB + prow + k * PR;
    const bool ok = pos < static_cast<uint32_t>(a.P);
    const size_t off = static_cast<size_t>(ok ? pos : sp * a.PB) * a.C;
    const RawVec<T, VEC> xv = load_raw<T, VEC>(x + off);
    const RawVec<T, VEC> dv = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + off));
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int ju = INSTANCE ? j : 0;
      const float xh = norm_elem<T, VEC>(xv, j, mean[ju], istd[ju], nmi[ju]);
      sdx[j] = elem_fma<T, VEC>(dv, j, xh, sdx[j]);
      sdy[j] = elem_fma<T, VEC>(dv, j, a.one, sdy[j]);
    }
  }
  split_pair_sums<TPR, VEC>(sdx, sdy, cvx, fold, chs);
}

// ---------------------------------------------------------------------------
// Backward.  With xh = (x-mean)*istd, per unit: s1 = sum gamma*dy,
// t2 = sum gamma*dy*xh (over the unit's channels and all positions),
//   cA = -istd*t2/R + 2*dvar*std/R,  cb = -s1*istd/R + dmean/R,
//   dx = gamma*istd*dy + cA*xh + cb
// (gn_cl_row_bwd_kernel / in_cl_row_bwd_kernel).  A block reduces the
// per-channel pairs (sum dy*xh, sum dy) of its positions, stores them for the
// batch sum behind dgamma/dbeta as "sample" n * split + s, publishes the
// partial (t2, s1) of each unit, collects its partners' and writes its dx.
// x stays in registers, dy is parked in LDS (each thread reads back what it
// wrote): both in registers cost more than the 128 a thread may use with two
// blocks of 512 on a CU.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int NL, int TPR, bool INSTANCE, bool MANY = false>
__global__ void __launch_bounds__(TPR, 4)
cl_split_bwd_kernel(const ClSplitArgs a) {
  constexpr int TV = kSplitTV;
  constexpr int PR = TPR / TV;
  constexpr int NW = TPR / kWave;
  constexpr int CH = TV * VEC; // channels of the tile
  constexpr int UMAX = INSTANCE ? CH : TV;
  constexpr int SV = INSTANCE ? VEC : 1; // statistics units of a thread's vector
  __shared__ RawVec<T, VEC> park[NL * TPR];
  __shared__ float fold[NW][2 * CH];
  __shared__ float chs[2][CH]; // [0]: sum dy*xh, [1]: sum dy per channel of the tile
  __shared__ float part16[MANY ? 1 : 16 * UMAX * 2];
  extern __shared__ float part_many[]; // [split][2 * units of the tile], sized by the launch
  float *const part = MANY ? part_many : part16;
  __shared__ float coef[UMAX * 2]; // (cA, cb) per unit
  __shared__ float gch[CH];        // gamma of the tile's channels
  __shared__ int missing[kSplitMax + 1];
  uint32_t tile, s, n;
  split_block_coords(a, blockIdx.x, tile, s, n);
  const uint32_t cvx = threadIdx.x % TV, prow = threadIdx.x / TV;
  const uint32_t ch0 = tile * CH, ch = ch0 + cvx * VEC;
  const uint32_t gi = INSTANCE ? 0u : (cvx >> a.cvg_shift);
  const int U = INSTANCE ? CH : (TV >> a.cvg_shift);
  const int per = 2 * U;
  const size_t slab = static_cast<size_t>(n) * a.P * a.C + ch;
  const T *__restrict__ x = static_cast<const T *>(a.x) + slab;
  const T *__restrict__ dy = static_cast<const T *>(a.dy) + slab;
  T *__restrict__ dx = a.out ? static_cast<T *>(a.out) + slab : nullptr;
  unsigned long long *slots =
      a.xchg + (static_cast<size_t>(n) * a.tiles + tile) * a.split * per;
  // statistics index of this thread's first unit
  const size_t stat = INSTANCE ? static_cast<size_t>(n) * a.C + ch
                               : static_cast<size_t>(n) * (a.C / a.cpg) + ch0 / a.cpg + gi;

  if (threadIdx.x <= kSplitMax) missing[threadIdx.x] = 0;
  // Small loads first, so that they travel with the tensor's: the thread's
  // statistics, gamma of channel threadIdx.x of the tile, and what the thread
  // of unit threadIdx.x needs for the unit's coefficients.
  float mean[SV], uvar[SV];
#pragma unroll
  for (int j = 0; j < SV; ++j) {
    mean[j] = a.mean[stat + j];
    uvar[j] = a.var[stat + j];
  }
  const bool unit_thread = static_cast<int>(threadIdx.x) < U;
  const size_t ustat = INSTANCE ? static_cast<size_t>(n) * a.C + ch0 + threadIdx.x
                                : static_cast<size_t>(n) * (a.C / a.cpg) + ch0 / a.cpg + threadIdx.x;
  float g_c = 1.f, u_var = 1.f, u_dvar = 0.f, u_dmean = 0.f;
  if (threadIdx.x < CH && a.gamma) g_c = a.gamma[ch0 + threadIdx.x];
  if (unit_thread) {
    u_var = a.var[ustat];
    if (a.dvar) u_dvar = a.dvar[ustat];
    if (a.dmean) u_dmean = a.dmean[ustat];
  }
  RawVec<T, VEC> xr[NL];
  {
    RawVec<T, VEC> dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const uint32_t pos = s * a.PB + prow + k * PR;
      const bool ok = pos < static_cast<uint32_t>(a.P);
      const size_t off = static_cast<size_t>(ok ? pos : s * a.PB) * a.C;
      xr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + off));
      dr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + off));
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) park[k * TPR + threadIdx.x] = dr[k];
  }
  float istd[SV], nmi[SV];
  // (An instance's VEC statistics per thread through LDS from the unit threads'
  // coalesced loads need a barrier here, in front of the first sums: [16,64,64,256]
  // half 25.1 -> 26.6 us; taken in 16-byte loads per thread: 25.4 -> 26.5 us.)
#pragma unroll
  for (int j = 0; j < SV; ++j) {
    istd[j] = 1.0f / sqrtf(uvar[j] + a.eps);
    nmi[j] = -mean[j] * istd[j];
  }
  if (threadIdx.x < CH) gch[threadIdx.x] = g_c; // (read behind the barriers of the first fold)

  // chs -> the partial (t2, s1) of every unit of the tile, into part[sp]
  auto unit_partials = [&](uint32_t sp, bool publish) {
    for (int e = threadIdx.x; e < per; e += TPR) {
      const int u = e >> 1, w = e & 1; // w = 0: t2 (from sum dy*xh), 1: s1 (from sum dy)
      float v;
      if constexpr (INSTANCE) {
        v = chs[w][u];
      } else {
        v = 0.f;
        for (int c = 0; c < a.cpg; ++c) {
          v = fmaf(gch[u * a.cpg + c], chs[w][u * a.cpg + c], v);
        }
      }
      part[sp * per + e] = v;
      if (publish) xchg_publish(slots + sp * per + e, v, a.epoch);
    }
  };

  // ---- this block's positions (own LDS entries only: no barrier needed before)
  {
    float sdx[VEC], sdy[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) sdx[j] = sdy[j] = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RawVec<T, VEC> dv = park[k * TPR + threadIdx.x];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const int ju = INSTANCE ? j : 0;
        const float xh = norm_elem<T, VEC>(xr[k], j, mean[ju], istd[ju], nmi[ju]);
        sdx[j] = elem_fma<T, VEC>(dv, j, xh, sdx[j]);
        sdy[j] = elem_fma<T, VEC>(dv, j, a.one, sdy[j]);
      }
    }
    split_pair_sums<TPR, VEC>(sdx, sdy, cvx, fold, chs);
    if (a.pairs) {
      for (int e = threadIdx.x; e < 2 * CH; e += TPR) {
        const int c = e >> 1, w = e & 1;
        a.pairs[2 * ((static_cast<size_t>(n) * a.split + s) * a.C + ch0 + c) + w] = chs[w][c];
      }
    }
    unit_partials(s, true);
  }
  if (dx == nullptr) return;

  // ---- the partners' parts
  split_collect<TPR>(a, slots, s, per, part, missing);
  lds_barrier();
  const bool any_missing = missing[kSplitMax] != 0; // (a flag per partner costs an LDS round trip each)
  for (int sp = 0; any_missing && sp < a.split; ++sp) {
    if (sp == static_cast<int>(s) || !missing[sp]) continue; // same answer in every thread
    // Partner sp has not published: its sums from global memory, a vector at a time.
    split_pairs_from_memory<T, VEC, NL, TPR, INSTANCE, SV>(a, x, dy, sp, prow, cvx, mean, istd, nmi,
                                                           fold, chs);
    unit_partials(static_cast<uint32_t>(sp), false);
    lds_barrier();
  }

  // ---- totals in block order and the unit's coefficients (a thread per unit), dx
  if (unit_thread) {
    const int u = static_cast<int>(threadIdx.x);
    float t2 = 0.f, s1 = 0.f;
    for_pairs_in_order(part + 2 * u, per, a.split, [&](int, float p0, float p1) {
      t2 += p0;
      s1 += p1;
    });
    if constexpr (INSTANCE) { // the exchanged sums are per channel, without gamma
      t2 *= g_c;
      s1 *= g_c;
    }
    const float vpe = u_var + a.eps;
    const float is = 1.0f / sqrtf(vpe);
    coef[2 * u] = -is * t2 * a.inv_R + (a.dvar ? 2.f * u_dvar * (vpe * is) * a.inv_R : 0.f);
    coef[2 * u + 1] = -s1 * is * a.inv_R + (a.dmean ? u_dmean * a.inv_R : 0.f);
  }
  lds_barrier();
#pragma unroll
  for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(xr[k]);
  // half: dx = dy*gis + x*A2 + B2 with A2 = istd*cA, B2 = nmi*cA + cb, two
  // mixed-precision fmas per element; float: dx = dy*gis + xh*cA + cb
  float gis[VEC], cA[SV], cb[SV];
#pragma unroll
  for (int j = 0; j < VEC; ++j) gis[j] = gch[cvx * VEC + j] * istd[INSTANCE ? j : 0];
#pragma unroll
  for (int j = 0; j < SV; ++j) {
    const int u = INSTANCE ? static_cast<int>(cvx) * VEC + j : static_cast<int>(gi);
    const float ca = coef[2 * u], cbu = coef[2 * u + 1];
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
    const uint32_t pos = s * a.PB + prow + k * PR;
    if (pos < static_cast<uint32_t>(a.P)) {
      const RawVec<T, VEC> dv = park[k * TPR + threadIdx.x];
      float o[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const int ju = INSTANCE ? j : 0;
        if constexpr (sizeof(T) == 2) {
          o[j] = elem_fma<T, VEC>(dv, j, gis[j], elem_fma<T, VEC>(xr[k], j, cA[ju], cb[ju]));
        } else {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean[ju], istd[ju], nmi[ju]);
          o[j] = elem_fma<T, VEC>(dv, j, gis[j], fmaf(xh, cA[ju], cb[ju]));
        }
      }
      T *p = dx + static_cast<size_t>(pos) * a.C;
      if (a.accum_dx) {
        float old[VEC];
        load_vec<T, VEC>(p, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] += old[j];
      }
      store_vec<T, VEC>(p, o);
    }
  }
}

} // namespace nblahip
