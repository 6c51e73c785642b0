// BatchNormalization kernels.  The tensor is [size0, C, size2]; one channel's
// N = size0*size2 values never fit on chip, so both directions are split
// reductions:
//   forward : stats partials (Welford per block) -> finalize (Chan merge,
//             running stats, per-channel apply parameters) -> apply
//   backward: (sum dy, sum dy*(x-mean)) partials -> finalize (dgamma, dbeta,
//             per-channel dx coefficients) -> apply
// Partials are merged in a fixed order (no atomics): results are reproducible.
//
// Two memory layouts get their own reduction kernels:
//   "planes"       size2 > 1 : a block owns one channel and a slice of its
//                  size0 planes; lanes run along the contiguous plane.
//   "channel-last" size2 == 1: x is [M, C]; a lane owns VEC adjacent channels,
//                  TX lanes span a row segment, TY = 256/TX rows per step.
#pragma once

#include "common.cuh"

namespace nblahip {

constexpr int kBnBlock = 256;
constexpr int kBnUnroll = 4; // 16-byte loads in flight per thread and input

// Per-channel parameters of the forward apply step: y = (x - mean)*scale + shift.
// Per-channel parameters of the backward apply step:
//   dx = c1*dy + c2*(x - mean) + c3.
struct __align__(16) BnParam {
  float mean, a, b, c;
};

// What a channel's finished statistics turn into (shared by the finalize
// kernel and by reduction blocks that own a whole channel):
//   mean, var (biased) -> batch_mean/batch_var
//   running mean/var update (unbiased N/(N-1) factor on the running variance,
//   the reference's kernel/batch_normalization.cuh:292-302)
//   apply parameters {mean, gamma*istd, beta}.
struct BnFwdFinal {
  float inv_N, unbias, decay, eps;
  const float *gamma, *beta;
  float *batch_mean, *batch_var, *rmean, *rvar;
  BnParam *params;
  __device__ __forceinline__ void publish(uint32_t c, const Welford &w) const {
    const float mean = w.mean;
    const float var = w.m2 * inv_N;
    batch_mean[c] = mean;
    batch_var[c] = var;
    if (rmean) rmean[c] = decay * rmean[c] + (1.f - decay) * mean;
    if (rvar) rvar[c] = decay * rvar[c] + (1.f - decay) * var * unbias;
    BnParam q;
    q.mean = mean;
    q.a = (gamma ? gamma[c] : 1.f) * inv_std(var, eps);
    q.b = beta ? beta[c] : 0.f;
    q.c = 0.f;
    params[c] = q;
  }
};

// Backward counterpart.  With sdx = sum dy*(x-mean), sdy = sum dy, g = gamma,
// i = istd (kernel/batch_normalization.cuh:425-469,522-540):
//   dgamma = sdx*i, dbeta = sdy
//   dvar   = -1/2 * g*sdx * i^3 + dv_in        dmean = -g*sdy*i + dm_in
//   dx     = g*i*dy + (2*dvar/N)*(x-mean) + dmean/N
// (the reference's dvar*(-2)*sum(x-mean)/N term vanishes identically).
// batch_stat == 0: statistics are constants, dx = g*i*dy.
struct BnBwdFinal {
  float inv_N, eps;
  int batch_stat;
  const float *gamma, *mean, *var, *dmean_in, *dvar_in;
  float *dgamma, *dbeta;
  int accum_g, accum_b;
  BnParam *params;
  // Optional: the channel's raw pair (sum dy*(x-mean), sum dy), for callers that
  // add the pairs of several shards of the batch before the apply step.
  float *sums;
  __device__ __forceinline__ void publish(uint32_t c, float sdx, float sdy) const {
    if (sums) {
      sums[2 * c] = sdx;
      sums[2 * c + 1] = sdy;
    }
    const float istd = inv_std(var[c], eps);
    const float g = gamma ? gamma[c] : 1.f;
    if (dgamma) dgamma[c] = sdx * istd + (accum_g ? dgamma[c] : 0.f);
    if (dbeta) dbeta[c] = sdy + (accum_b ? dbeta[c] : 0.f);
    BnParam q;
    q.mean = mean[c];
    q.a = g * istd;
    if (batch_stat) {
      const float dvar = -0.5f * g * sdx * istd * istd * istd + (dvar_in ? dvar_in[c] : 0.f);
      const float dmean = -g * sdy * istd + (dmean_in ? dmean_in[c] : 0.f);
      q.b = 2.f * dvar * inv_N;
      q.c = dmean * inv_N;
    } else {
      q.b = 0.f;
      q.c = 0.f;
    }
    params[c] = q;
  }
};

// Offset (in vectors) of vector v of channel c in the planes layout.
__device__ __forceinline__ size_t bn_plane_offset(uint32_t v, uint32_t c, uint32_t C,
                                                  const FastDiv &nvp) {
  const uint32_t n = nvp.div(v);
  const uint32_t i = v - n * nvp.d;
  return (static_cast<size_t>(n) * C + c) * nvp.d + i;
}

// A plane whose length is no multiple of the vector width: the kernels still
// use vectors aligned in the TENSOR (base pointers 16-byte aligned, element
// count a multiple of VEC), and a plane is covered by the nvp = ceil((VEC - 1 +
// size2) / VEC) aligned vectors that can overlap it; elements of a vector
// outside the plane (they belong to the neighbouring channels) are masked.
// PlaneVec: element offset of the vector and the range [lo, hi) of its
// elements that lie in the plane.
struct PlaneVec {
  size_t off;
  int lo, hi;
};

template <int VEC, bool MASKED>
__device__ __forceinline__ PlaneVec bn_plane_vec(uint32_t v, uint32_t c, uint32_t C,
                                                 const FastDiv &nvp, uint32_t size2,
                                                 uint32_t last_vec) {
  PlaneVec r;
  if constexpr (!MASKED) {
    r.off = bn_plane_offset(v, c, C, nvp) * VEC;
    r.lo = 0;
    r.hi = VEC;
  } else {
    const uint32_t n = nvp.div(v);
    const uint32_t i = v - n * nvp.d;
    const uint32_t first = (n * C + c) * size2; // first element of the plane
    r.lo = static_cast<int>(first % VEC) - static_cast<int>(i * VEC);
    r.hi = r.lo + static_cast<int>(size2);
    // A vector past the plane's end has hi <= 0 (nothing valid); keep its
    // address inside the tensor.
    r.off = static_cast<size_t>(min(first / VEC + i, last_vec)) * VEC;
  }
  return r;
}

// ---------------------------------------------------------------------------
// Forward statistics, planes layout.  grid = (C, S).
// vpc = vectors per channel = size0 * nvp; split s covers vectors
// [s*chunk, min((s+1)*chunk, vpc)).  DIRECT (S == 1, BLOCK = 1024): the block
// owns the whole channel and publishes its statistics itself; used when there
// are enough channels to give every CU a block, which removes the partial
// buffer and the finalize launch.  U = 16-byte loads in flight per thread.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int BLOCK, bool DIRECT, int U, bool MASKED = false>
__global__ void __launch_bounds__(BLOCK)
bn_stats_planes_kernel(const T *__restrict__ x, uint32_t C, FastDiv nvp, uint32_t vpc,
                       uint32_t chunk, float *__restrict__ part /*[C][S][3]*/, BnFwdFinal fin,
                       uint32_t size2, uint32_t last_vec) {
  __shared__ float lds[3 * (BLOCK / kWave)];
  const uint32_t c = blockIdx.x;
  const uint32_t s = blockIdx.y;
  const uint32_t S = gridDim.y;
  const uint32_t begin = s * chunk;
  const uint32_t end = min(begin + chunk, vpc);
  Welford w{0.f, 0.f, 0.f};
  uint32_t v0 = begin + threadIdx.x;
  if constexpr (MASKED) {
    for (; v0 < end; v0 += BLOCK * U) {
      RawVec<T, VEC> raw[U];
      PlaneVec pv[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * BLOCK;
        pv[u] = bn_plane_vec<VEC, true>(v < end ? v : v0, c, C, nvp, size2, last_vec);
        raw[u] = load_raw<T, VEC>(x + pv[u].off);
        if (v >= end) pv[u].hi = pv[u].lo;
      }
      float vals[U * VEC];
      bool ok[U * VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float tmp[VEC];
        unpack<T, VEC>(raw[u], tmp);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          ok[u * VEC + j] = j >= pv[u].lo && j < pv[u].hi;
          vals[u * VEC + j] = tmp[j];
        }
      }
      welford_add_chunk_masked<U * VEC>(w, vals, ok);
    }
  }
  // full steps: every load valid, all U loads in flight together
  for (; !MASKED && v0 + (U - 1) * BLOCK < end; v0 += BLOCK * U) {
    RawVec<T, VEC> raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      raw[u] = load_raw<T, VEC>(x + bn_plane_offset(v0 + u * BLOCK, c, C, nvp) * VEC);
    float vals[U * VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float tmp[VEC];
      unpack<T, VEC>(raw[u], tmp);
#pragma unroll
      for (int j = 0; j < VEC; ++j) vals[u * VEC + j] = tmp[j];
    }
    welford_add_chunk<U * VEC>(w, vals, U * VEC);
  }
  if (!MASKED && v0 < end) { // ragged last step: clamp the index, count what is real
    float vals[U * VEC];
    int cnt = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t v = v0 + u * BLOCK;
      const bool ok = v < end;
      float tmp[VEC];
      unpack<T, VEC>(load_raw<T, VEC>(x + bn_plane_offset(ok ? v : v0, c, C, nvp) * VEC), tmp);
#pragma unroll
      for (int j = 0; j < VEC; ++j) vals[u * VEC + j] = ok ? tmp[j] : 0.f;
      cnt += ok ? VEC : 0;
    }
    welford_add_chunk<U * VEC>(w, vals, cnt);
  }
  w = block_welford(w, lds);
  if (threadIdx.x == 0) {
    if constexpr (DIRECT) {
      fin.publish(c, w);
    } else {
      float *p = part + 3 * (static_cast<size_t>(c) * S + s);
      p[0] = w.mean;
      p[1] = w.m2;
      p[2] = w.n;
    }
  }
}

// ---------------------------------------------------------------------------
// Forward statistics, channel-last layout x[M][C].  grid = (ceil(ncv/TX), S),
// ncv = C/VEC.  Split s covers rows [s*rps, min((s+1)*rps, M)).
// A thread keeps VEC Welford states (one per channel it owns) and feeds them
// chunks of kBnClRows rows: chunk mean, centred chunk M2, one Chan merge.
// ---------------------------------------------------------------------------
constexpr int kBnClRows = 8;

template <typename T, int VEC, bool FULL>
__device__ __forceinline__ void bn_cl_chunk(const RawVec<T, VEC> (&raw)[kBnClRows], int cnt,
                                            float one, float (&mean)[VEC], float (&m2)[VEC],
                                            float &n) {
  const float fc = static_cast<float>(cnt);
  const float inv_fc = fast_rcp(fc);
  const float nn = n + fc;
  const float wb = fc * fast_rcp(nn); // weight of the chunk mean
  const float wd = n * wb;            // n_a*n_b/(n_a+n_b)
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    float sum = 0.f; // rows beyond cnt were zeroed at load time
#pragma unroll
    for (int u = 0; u < kBnClRows; ++u) sum = elem_fma<T, VEC>(raw[u], j, one, sum);
    const float cm = sum * inv_fc;
    float cm2 = 0.f;
#pragma unroll
    for (int u = 0; u < kBnClRows; ++u) {
      const float d = elem_fma<T, VEC>(raw[u], j, one, -cm);
      if (FULL || u < cnt) cm2 = fmaf(d, d, cm2);
    }
    const float d = cm - mean[j];
    mean[j] = fmaf(d, wb, mean[j]);
    m2[j] += fmaf(d * d, wd, cm2);
  }
  n = nn;
}

template <typename T, int VEC>
__global__ void __launch_bounds__(kBnBlock)
bn_stats_cl_kernel(const T *__restrict__ x, uint32_t M, uint32_t C, uint32_t ncv,
                   uint32_t log2tx, uint32_t rps, float one,
                   float *__restrict__ part /*[C][S][3]*/) {
  // [TY][TX*VEC] means and m2 plus [TY][TX] counts; TY*TX == 256.
  __shared__ float lmean[kBnBlock * VEC];
  __shared__ float lm2[kBnBlock * VEC];
  __shared__ float ln[kBnBlock];
  __shared__ float l2[3 * kBnBlock]; // second merge level: [q][o] triples
  const uint32_t TX = 1u << log2tx;
  const uint32_t TY = kBnBlock >> log2tx;
  const uint32_t tx = threadIdx.x & (TX - 1);
  const uint32_t ty = threadIdx.x >> log2tx;
  const uint32_t cv = blockIdx.x * TX + tx;
  const bool active = cv < ncv;
  const uint32_t S = gridDim.y;
  const uint32_t s = blockIdx.y;
  const uint32_t rbegin = s * rps;
  const uint32_t rend = min(rbegin + rps, M);
  // blockIdx.z: independent [M, C] slabs (the samples of a channel-last
  // Group/InstanceNormalization); BatchNormalization launches one slab.
  x += static_cast<size_t>(blockIdx.z) * M * C;
  part += static_cast<size_t>(blockIdx.z) * C * S * 3;

  float mean[VEC], m2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] = m2[j] = 0.f;
  float n = 0.f;

  if (active) {
    const T *xc = x + static_cast<size_t>(cv) * VEC;
    uint32_t r0 = rbegin + ty;
    // full chunks: every row valid, no masks
    for (; r0 + (kBnClRows - 1) * TY < rend; r0 += TY * kBnClRows) {
      RawVec<T, VEC> raw[kBnClRows];
#pragma unroll
      for (int u = 0; u < kBnClRows; ++u)
        raw[u] = load_raw<T, VEC>(xc + static_cast<size_t>(r0 + u * TY) * C);
      bn_cl_chunk<T, VEC, true>(raw, kBnClRows, one, mean, m2, n);
    }
    if (r0 < rend) { // tail chunk: clamp the row, zero what lies beyond
      RawVec<T, VEC> raw[kBnClRows];
      int cnt = 0;
#pragma unroll
      for (int u = 0; u < kBnClRows; ++u) {
        const uint32_t r = r0 + u * TY;
        const bool ok = r < rend;
        raw[u] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(xc + static_cast<size_t>(ok ? r : r0) * C));
        cnt += ok ? 1 : 0;
      }
      bn_cl_chunk<T, VEC, false>(raw, cnt, one, mean, m2, n);
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    lmean[(ty * TX + tx) * VEC + j] = mean[j];
    lm2[(ty * TX + tx) * VEC + j] = m2[j];
  }
  ln[ty * TX + tx] = n;
  lds_barrier();
  // Output o = tx*VEC + j of this block needs its TY row groups folded.  With
  // nout = TX*VEC outputs and 256 threads, Q = 256/nout threads share an
  // output: each folds TY/Q row groups in order, then the Q results are
  // folded in order by the first of them (fixed order: reproducible).
  const uint32_t nout = TX * VEC;
  if (nout <= kBnBlock) {
    const uint32_t Q = kBnBlock / nout;
    const uint32_t per = (TY + Q - 1) / Q;
    const uint32_t o = threadIdx.x % nout;
    const uint32_t q = threadIdx.x / nout;
    const uint32_t otx = o / VEC;
    Welford w{0.f, 0.f, 0.f};
    for (uint32_t y = q * per; y < min((q + 1) * per, TY); ++y) {
      const Welford b{lmean[y * nout + o], lm2[y * nout + o], ln[y * TX + otx]};
      w = welford_merge(w, b);
    }
    l2[3 * threadIdx.x] = w.mean;
    l2[3 * threadIdx.x + 1] = w.m2;
    l2[3 * threadIdx.x + 2] = w.n;
    lds_barrier();
    if (q == 0 && blockIdx.x * TX + otx < ncv) {
      for (uint32_t k = 1; k < Q; ++k) {
        const uint32_t t = k * nout + o;
        w = welford_merge(w, Welford{l2[3 * t], l2[3 * t + 1], l2[3 * t + 2]});
      }
      const uint32_t ch = blockIdx.x * nout + o;
      float *p = part + 3 * (static_cast<size_t>(ch) * S + s);
      p[0] = w.mean;
      p[1] = w.m2;
      p[2] = w.n;
    }
  } else {
    for (uint32_t o = threadIdx.x; o < nout; o += kBnBlock) {
      const uint32_t otx = o / VEC;
      if (blockIdx.x * TX + otx < ncv) {
        Welford w{0.f, 0.f, 0.f};
        for (uint32_t y = 0; y < TY; ++y) {
          const Welford b{lmean[y * nout + o], lm2[y * nout + o], ln[y * TX + otx]};
          w = welford_merge(w, b);
        }
        const uint32_t ch = blockIdx.x * nout + o;
        float *p = part + 3 * (static_cast<size_t>(ch) * S + s);
        p[0] = w.mean;
        p[1] = w.m2;
        p[2] = w.n;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Forward finalize: one block per channel merges its S partials.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBnBlock)
bn_finalize_fwd_kernel(const float *__restrict__ part, uint32_t S, BnFwdFinal fin) {
  __shared__ float lds[3 * (kBnBlock / kWave)];
  const uint32_t c = blockIdx.x;
  Welford w{0.f, 0.f, 0.f};
  for (uint32_t s = threadIdx.x; s < S; s += kBnBlock) {
    const float *p = part + 3 * (static_cast<size_t>(c) * S + s);
    w = welford_merge(w, Welford{p[0], p[1], p[2]});
  }
  w = block_welford(w, lds);
  if (threadIdx.x == 0) fin.publish(c, w);
}

// How the apply kernels obtain a channel's parameters.
//   params != null : precomputed by a finalize kernel
//   params == null : inference, computed on the fly from running statistics
struct BnParamSrc {
  const BnParam *params;
  const float *rmean, *rvar, *gamma, *beta;
  float eps;
  __device__ __forceinline__ BnParam get(uint32_t c) const {
    if (params) return params[c];
    BnParam q;
    q.mean = rmean ? rmean[c] : 0.f; // (no mean: the inference-mode backward, dx = dy * a)
    q.a = (gamma ? gamma[c] : 1.f) * inv_std(rvar[c], eps);
    q.b = beta ? beta[c] : 0.f;
    q.c = 0.f;
    return q;
  }
};

// ---------------------------------------------------------------------------
// Forward apply, planes layout, flattened over all vectors of the tensor.
// plane = i / nvp, c = plane % C.
// ---------------------------------------------------------------------------
// FUSE (FusedBatchNormalization): 0 plain, 1 y = max(0, bn), 2 y = max(0, bn + z).
// STRADDLE: planes of nvp.d ELEMENTS (>= VEC, no multiple of VEC); a vector
// then holds the end of one plane and the start of the next at most, and each
// element picks the parameters of its own channel.
// The parameters of the planes a block step meets (one per vector at most, and
// the plane after a straddling vector's) go through LDS, each computed by one
// thread: taken per vector they cost the inference path four loads and a
// division by a square root each time, more than the vector's own traffic.
constexpr uint32_t kApplyStep = 256u * kBnUnroll;
constexpr uint32_t kApplyTab = kApplyStep + 4;

template <typename T, int VEC, int FUSE = 0, bool STRADDLE = false>
__global__ void __launch_bounds__(256)
bn_apply_planes_kernel(const T *__restrict__ x, T *__restrict__ y, BnParamSrc src,
                       FastDiv nvp, FastDiv cdiv, uint32_t total_vec,
                       const T *__restrict__ z) {
  __shared__ float tab[3 * kApplyTab];
  for (uint32_t vb = blockIdx.x * kApplyStep; vb < total_vec; vb += gridDim.x * kApplyStep) {
    const uint32_t i0 = vb + threadIdx.x;
    float v[kBnUnroll][VEC];
    float zv[FUSE == 2 ? kBnUnroll : 1][VEC];
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      const uint32_t i = i0 + u * 256u;
      if (i < total_vec) {
        load_vec<T, VEC>(x + static_cast<size_t>(i) * VEC, v[u]);
        if constexpr (FUSE == 2) load_vec<T, VEC>(z + static_cast<size_t>(i) * VEC, zv[u]);
      }
    }
    const uint32_t ve = min(vb + kApplyStep, total_vec) - 1;
    const uint32_t p0 = nvp.div(STRADDLE ? vb * VEC : vb);
    const uint32_t p1 = STRADDLE ? nvp.div(ve * VEC + (VEC - 1)) + 1 : nvp.div(ve);
    __syncthreads(); // the step before has read its table
    for (uint32_t k = threadIdx.x; k <= p1 - p0; k += 256u) {
      const uint32_t plane = p0 + k;
      const BnParam q = src.get(plane - cdiv.div(plane) * cdiv.d);
      tab[k] = q.mean;
      tab[kApplyTab + k] = q.a;
      tab[2 * kApplyTab + k] = q.b;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      const uint32_t i = i0 + u * 256u;
      if (i < total_vec) {
        const uint32_t plane = nvp.div(STRADDLE ? i * VEC : i);
        const uint32_t k = plane - p0;
        const float qm = tab[k], qa = tab[kApplyTab + k], qb = tab[2 * kApplyTab + k];
        float o[VEC];
        if constexpr (STRADDLE) {
          // elements j >= cross belong to the next plane
          const int cross = static_cast<int>(nvp.d - (i * VEC - plane * nvp.d));
          const float nm = tab[k + 1], na = tab[kApplyTab + k + 1], nb = tab[2 * kApplyTab + k + 1];
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const bool nx = j >= cross;
            o[j] = (v[u][j] - (nx ? nm : qm)) * (nx ? na : qa) + (nx ? nb : qb);
          }
        } else if constexpr (sizeof(T) == 2) {
          // Half output: one mixed-precision fma per element; the folded shift
          // loses nothing a 10-bit mantissa can hold.
          const float shift = fmaf(-qm, qa, qb);
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = fmaf(v[u][j], qa, shift);
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = (v[u][j] - qm) * qa + qb;
        }
        if constexpr (FUSE == 2) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] += zv[u][j];
        }
        if constexpr (FUSE != 0) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = fmaxf(0.f, o[j]);
        }
        store_vec<T, VEC>(y + static_cast<size_t>(i) * VEC, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Thread layout of the channel-last apply kernels over a slab x[M][ncv] of
// vectors: a thread always meets the same VEC channels, so their parameters
// live in registers.  A block covers cols = min(ncv, 256) channel vectors of
// R = 256 / cols rows per step (threads past R*cols idle; for ncv dividing 256
// there are none and the block walks the slab as one contiguous run).  Wider
// rows are cut into ntiles = ceil(ncv / 256) column tiles;
// gridDim.x = ntiles * row blocks.  (Narrower tiles, tile_cols a power of two:
// fewer channels per block to prepare.)
// ---------------------------------------------------------------------------
struct ClApplyMap {
  uint32_t cv;       // channel vector of this thread
  uint32_t col;      // ... counted from the tile's first
  uint32_t row0;     // first row
  uint32_t R;        // rows between the U loads of one step
  uint32_t row_step; // rows between steps
  bool active;
};

template <int U>
__device__ __forceinline__ ClApplyMap cl_apply_map(uint32_t ncv, uint32_t ntiles,
                                                   uint32_t tile_cols = 256u) {
  ClApplyMap m;
  const uint32_t cols = min(ncv, tile_cols);
  m.R = 256u / cols;
  const uint32_t tr = threadIdx.x / cols;
  const uint32_t tile = blockIdx.x % ntiles;
  const uint32_t rb = blockIdx.x / ntiles;
  m.col = threadIdx.x - tr * cols;
  m.cv = tile * tile_cols + m.col;
  m.active = tr < m.R && m.cv < ncv;
  m.row0 = rb * m.R * U + tr;
  m.row_step = (gridDim.x / ntiles) * m.R * U;
  return m;
}

// ---------------------------------------------------------------------------
// Forward apply, channel-last.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int FUSE = 0>
__global__ void __launch_bounds__(256)
bn_apply_cl_kernel(const T *__restrict__ x, T *__restrict__ y, BnParamSrc src,
                   uint32_t ncv, uint32_t ntiles, uint32_t M, const T *__restrict__ z,
                   float one, uint32_t tile_cols) {
  // blockIdx.y: slab (sample) index; each slab has its own ncv*VEC parameters.
  const size_t slab = static_cast<size_t>(blockIdx.y) * M * ncv * VEC;
  x += slab;
  y += slab;
  if constexpr (FUSE == 2) z += slab;
  if (src.params) src.params += static_cast<size_t>(blockIdx.y) * ncv * VEC;
  const ClApplyMap map = cl_apply_map<kBnUnroll>(ncv, ntiles, tile_cols);
  // The parameters of the block's channels go through LDS, each computed by
  // one thread from coalesced loads: every thread taking its own VEC channels
  // costs the inference path 4*VEC strided loads and VEC divisions by a square
  // root per thread, which the texture path serializes over the block.
  __shared__ float tab[3 * 256 * VEC];
  {
    const uint32_t c0 = (blockIdx.x % ntiles) * tile_cols * VEC;
    const uint32_t nch = min(tile_cols * VEC, ncv * VEC - c0);
    for (uint32_t k = threadIdx.x; k < nch; k += 256u) {
      const BnParam q = src.get(c0 + k);
      tab[k] = q.mean;
      tab[256 * VEC + k] = q.a;
      tab[2 * 256 * VEC + k] = (sizeof(T) == 2) ? fmaf(-q.mean, q.a, q.b) : q.b;
    }
    __syncthreads();
  }
  if (!map.active) return;
  const uint32_t cv = map.cv;
  // y = x*pa + ps with ps = pb - mean*pa for half output (one mixed fma per
  // element); the centred form (x-mean)*pa + pb for float output.
  float pm[VEC], pa[VEC], pb[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t k = map.col * VEC + j;
    pm[j] = tab[k];
    pa[j] = tab[256 * VEC + k];
    pb[j] = tab[2 * 256 * VEC + k];
  }
  for (uint32_t r0 = map.row0; r0 < M; r0 += map.row_step) {
    RawVec<T, VEC> raw[kBnUnroll];
    RawVec<T, VEC> zr[FUSE == 2 ? kBnUnroll : 1];
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      // clamped: loads stay branch-free
      const uint32_t i = min(r0 + u * map.R, M - 1) * ncv + cv;
      raw[u] = load_raw<T, VEC>(x + static_cast<size_t>(i) * VEC);
      if constexpr (FUSE == 2) zr[u] = load_raw<T, VEC>(z + static_cast<size_t>(i) * VEC);
    }
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      const uint32_t row = r0 + u * map.R;
      const uint32_t i = row * ncv + cv;
      if (row < M) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if constexpr (sizeof(T) == 2) {
            o[j] = elem_fma<T, VEC>(raw[u], j, pa[j], pb[j]);
          } else {
            o[j] = (elem_fma<T, VEC>(raw[u], j, 1.0f, 0.f) - pm[j]) * pa[j] + pb[j];
          }
          if constexpr (FUSE == 2) o[j] = elem_fma<T, VEC>(zr[u], j, one, o[j]);
          if constexpr (FUSE != 0) o[j] = fmaxf(0.f, o[j]);
        }
        store_vec<T, VEC>(y + static_cast<size_t>(i) * VEC, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Backward reduction, planes layout.  part2[C][S][2] = (sum dy*(x-mean), sum dy).
// DIRECT as in bn_stats_planes_kernel.
// ---------------------------------------------------------------------------
// FUSED (FusedBatchNormalization): dy is first masked by y > 0 (ReLU backward);
// the masked dy is stored to dz when dz != null (the gradient of the residual
// input, which the apply step can then read in place of dy and y).
template <typename T, int VEC, int BLOCK, bool DIRECT, bool FUSED = false, bool MASKED = false>
__global__ void __launch_bounds__(BLOCK)
bn_bwd_reduce_planes_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                            const float *__restrict__ mean, uint32_t C, FastDiv nvp,
                            uint32_t vpc, uint32_t chunk, float one, float *__restrict__ part2,
                            BnBwdFinal fin, const T *__restrict__ y, T *__restrict__ dz,
                            uint32_t size2, uint32_t last_vec) {
  __shared__ float lds[2 * (BLOCK / kWave)];
  const uint32_t c = blockIdx.x;
  const uint32_t s = blockIdx.y;
  const uint32_t S = gridDim.y;
  const uint32_t begin = s * chunk;
  const uint32_t end = min(begin + chunk, vpc);
  const float nm = -mean[c];
  float sdx = 0.f, sdy = 0.f;
  for (uint32_t v0 = begin + threadIdx.x; v0 < end; v0 += BLOCK * kBnUnroll) {
    RawVec<T, VEC> xr[kBnUnroll], dr[kBnUnroll];
    RawVec<T, VEC> yr[FUSED ? kBnUnroll : 1];
    PlaneVec pv[kBnUnroll];
    // all loads first (indices past the end re-read v0), selects after
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      const uint32_t v = v0 + u * BLOCK;
      pv[u] = bn_plane_vec<VEC, MASKED>(v < end ? v : v0, c, C, nvp, size2, last_vec);
      xr[u] = load_raw<T, VEC>(x + pv[u].off);
      dr[u] = load_raw<T, VEC>(dy + pv[u].off);
      if constexpr (FUSED) yr[u] = load_raw<T, VEC>(y + pv[u].off);
    }
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      dr[u] = raw_or_zero<T, VEC>(v0 + u * BLOCK < end, dr[u]);
      if constexpr (MASKED) dr[u] = raw_keep_range<T, VEC>(dr[u], pv[u].lo, pv[u].hi);
    }
    if constexpr (FUSED) {
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) dr[u] = raw_relu_mask<T, VEC>(dr[u], yr[u]);
      if (dz) {
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) {
          const uint32_t v = v0 + u * BLOCK;
          if (v < end) {
            if (!MASKED || (pv[u].lo <= 0 && pv[u].hi >= VEC)) {
              store_raw<T, VEC>(dz + pv[u].off, dr[u]);
            } else { // a vector shared with the neighbouring planes: element stores
              float g[VEC];
              unpack<T, VEC>(dr[u], g);
#pragma unroll
              for (int j = 0; j < VEC; ++j)
                if (j >= pv[u].lo && j < pv[u].hi) dz[pv[u].off + j] = from_f32<T>(g[j]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u) {
      sdy = raw_sum<T, VEC>(dr[u], sdy);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xc = elem_fma<T, VEC>(xr[u], j, one, nm);
        sdx = elem_fma<T, VEC>(dr[u], j, xc, sdx);
      }
    }
  }
  block_sum2(sdx, sdy, lds);
  if (threadIdx.x == 0) {
    if constexpr (DIRECT) {
      fin.publish(c, sdx, sdy);
    } else {
      float *p = part2 + 2 * (static_cast<size_t>(c) * S + s);
      p[0] = sdx;
      p[1] = sdy;
    }
  }
}

// ---------------------------------------------------------------------------
// Backward reduction, channel-last.  Same thread layout as bn_stats_cl_kernel.
// ---------------------------------------------------------------------------
template <typename T, int VEC, bool FUSED = false>
__global__ void __launch_bounds__(kBnBlock)
bn_bwd_reduce_cl_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                        const float *__restrict__ mean, uint32_t M, uint32_t C,
                        uint32_t ncv, uint32_t log2tx, uint32_t rps, float one,
                        float *__restrict__ part2 /*[C][S][2]*/, uint32_t mean_slab_stride,
                        FastDiv cpg, const T *__restrict__ y, T *__restrict__ dz) {
  __shared__ float lsdx[kBnBlock * VEC];
  __shared__ float lsdy[kBnBlock * VEC];
  const uint32_t TX = 1u << log2tx;
  const uint32_t TY = kBnBlock >> log2tx;
  const uint32_t tx = threadIdx.x & (TX - 1);
  const uint32_t ty = threadIdx.x >> log2tx;
  const uint32_t cv = blockIdx.x * TX + tx;
  const bool active = cv < ncv;
  const uint32_t S = gridDim.y;
  const uint32_t s = blockIdx.y;
  const uint32_t rbegin = s * rps;
  const uint32_t rend = min(rbegin + rps, M);

  float sdx[VEC], sdy[VEC], nm[VEC];
  {
    // Clamped index instead of a branch: one vector load of the VEC means.
    // Mean of channel c in slab z: mean[z*mean_slab_stride + c/cpg]
    // (BatchNormalization: stride 0, cpg 1; GroupNormalization: stride G,
    // cpg channels per group).
    x += static_cast<size_t>(blockIdx.z) * M * C;
    dy += static_cast<size_t>(blockIdx.z) * M * C;
    part2 += static_cast<size_t>(blockIdx.z) * C * gridDim.y * 2;
    mean += static_cast<size_t>(blockIdx.z) * mean_slab_stride;
    float mv[VEC];
    const uint32_t cvc = active ? cv : 0u;
#pragma unroll
    for (int j = 0; j < VEC; ++j) mv[j] = mean[cpg.div(cvc * VEC + j)];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      sdx[j] = sdy[j] = 0.f;
      nm[j] = -mv[j];
    }
  }
  if (active) {
    for (uint32_t r0 = rbegin + ty; r0 < rend; r0 += TY * kBnUnroll) {
      RawVec<T, VEC> xr[kBnUnroll], dr[kBnUnroll];
      RawVec<T, VEC> yr[FUSED ? kBnUnroll : 1];
      // All loads first (rows beyond the split re-read row r0), selects after:
      // the eight loads are in flight together.
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) {
        const uint32_t r = r0 + u * TY;
        const size_t off = static_cast<size_t>(r < rend ? r : r0) * C + static_cast<size_t>(cv) * VEC;
        xr[u] = load_raw<T, VEC>(x + off);
        dr[u] = load_raw<T, VEC>(dy + off);
        if constexpr (FUSED) yr[u] = load_raw<T, VEC>(y + off);
      }
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) // dy zeroed beyond the split: adds nothing
        dr[u] = raw_or_zero<T, VEC>(r0 + u * TY < rend, dr[u]);
      if constexpr (FUSED) {
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) dr[u] = raw_relu_mask<T, VEC>(dr[u], yr[u]);
        if (dz) {
#pragma unroll
          for (int u = 0; u < kBnUnroll; ++u) {
            const uint32_t r = r0 + u * TY;
            if (r < rend)
              store_raw<T, VEC>(dz + static_cast<size_t>(r) * C + static_cast<size_t>(cv) * VEC,
                                dr[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u)
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xc = elem_fma<T, VEC>(xr[u], j, one, nm[j]);
          sdy[j] = elem_fma<T, VEC>(dr[u], j, one, sdy[j]);
          sdx[j] = elem_fma<T, VEC>(dr[u], j, xc, sdx[j]);
        }
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    lsdx[(ty * TX + tx) * VEC + j] = sdx[j];
    lsdy[(ty * TX + tx) * VEC + j] = sdy[j];
  }
  lds_barrier();
  for (uint32_t o = threadIdx.x; o < TX * VEC; o += kBnBlock) {
    const uint32_t otx = o / VEC;
    const uint32_t ch = blockIdx.x * TX * VEC + o;
    if (blockIdx.x * TX + otx < ncv) {
      float a = 0.f, b = 0.f;
      for (uint32_t y = 0; y < TY; ++y) {
        a += lsdx[y * TX * VEC + o];
        b += lsdy[y * TX * VEC + o];
      }
      float *p = part2 + 2 * (static_cast<size_t>(ch) * S + s);
      p[0] = a;
      p[1] = b;
    }
  }
}

// ---------------------------------------------------------------------------
// Statistics of a batch that is split over `workers` shards (the exchange step
// of the reference's SyncBatchNormalization,
// batch_norm_reduce_statistics_kernel, kernel/sync_batch_normalization.cuh:
// 448-487): stats[w] = {mean[C], var[C] (biased, over the shard), count}.
// Chan merge in shard order -> mean/var of the whole batch, running statistics
// with the unbiased N/(N-1) factor on the total count.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
bn_merge_stats_kernel(const float *__restrict__ stats, uint32_t workers, uint32_t C,
                      float *__restrict__ batch_mean, float *__restrict__ batch_var,
                      float *__restrict__ rmean, float *__restrict__ rvar, float decay) {
  const uint32_t c = blockIdx.x * 256u + threadIdx.x;
  if (c >= C) return;
  const size_t stride = 2 * static_cast<size_t>(C) + 1;
  Welford w{0.f, 0.f, 0.f};
  for (uint32_t j = 0; j < workers; ++j) {
    const float *s = stats + j * stride;
    const float n = s[2 * C];
    w = welford_merge(w, Welford{s[c], s[C + c] * n, n});
  }
  const float var = w.n > 0.f ? w.m2 / w.n : 0.f;
  batch_mean[c] = w.mean;
  batch_var[c] = var;
  if (rmean) rmean[c] = decay * rmean[c] + (1.f - decay) * w.mean;
  if (rvar) rvar[c] = decay * rvar[c] + (1.f - decay) * (w.m2 / (w.n - 1.f));
}

// ---------------------------------------------------------------------------
// Backward finalize (one block per channel): sums the S partial pairs.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBnBlock)
bn_finalize_bwd_kernel(const float *__restrict__ part2, uint32_t S, BnBwdFinal fin) {
  __shared__ float lds[2 * (kBnBlock / kWave)];
  const uint32_t c = blockIdx.x;
  float sdx = 0.f, sdy = 0.f;
  for (uint32_t s = threadIdx.x; s < S; s += kBnBlock) {
    const float *p = part2 + 2 * (static_cast<size_t>(c) * S + s);
    sdx += p[0];
    sdy += p[1];
  }
  block_sum2(sdx, sdy, lds);
  if (threadIdx.x == 0) fin.publish(c, sdx, sdy);
}

// ---------------------------------------------------------------------------
// Backward apply: dx = a*dy + b*(x-mean) + c (+ dx).
// ---------------------------------------------------------------------------
// FUSED (FusedBatchNormalization): dy is first masked by y > 0; the masked dy
// is also the gradient of the residual input z (dz, optional).  dx may be
// null when FUSED (only dz wanted).
template <typename T, int VEC, bool FUSED = false, bool STRADDLE = false>
__global__ void __launch_bounds__(256)
bn_bwd_apply_planes_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                           T *__restrict__ dx, const BnParam *__restrict__ params,
                           FastDiv nvp, FastDiv cdiv, uint32_t total_vec, int accum,
                           const T *__restrict__ y, T *__restrict__ dz, int accum_dz) {
  constexpr int U = 2;
  for (uint32_t i0 = blockIdx.x * (256u * U) + threadIdx.x; i0 < total_vec;
       i0 += gridDim.x * (256u * U)) {
    float xv[U][VEC], dv[U][VEC];
    float yv[FUSED ? U : 1][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + u * 256u;
      if (i < total_vec) {
        load_vec<T, VEC>(x + static_cast<size_t>(i) * VEC, xv[u]);
        load_vec<T, VEC>(dy + static_cast<size_t>(i) * VEC, dv[u]);
        if constexpr (FUSED) load_vec<T, VEC>(y + static_cast<size_t>(i) * VEC, yv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + u * 256u;
      if (i < total_vec) {
        if constexpr (FUSED) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) dv[u][j] = yv[u][j] > 0.f ? dv[u][j] : 0.f;
          if (dz) {
            float g[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) g[j] = dv[u][j];
            if (accum_dz) {
              float old[VEC];
              load_vec<T, VEC>(dz + static_cast<size_t>(i) * VEC, old);
#pragma unroll
              for (int j = 0; j < VEC; ++j) g[j] += old[j];
            }
            store_vec<T, VEC>(dz + static_cast<size_t>(i) * VEC, g);
          }
          if (!dx) continue;
        }
        const uint32_t plane = nvp.div(STRADDLE ? i * VEC : i);
        const uint32_t c = plane - cdiv.div(plane) * cdiv.d;
        const BnParam q = params[c];
        float o[VEC];
        if constexpr (STRADDLE) { // as in bn_apply_planes_kernel
          const int cross = static_cast<int>(nvp.d - (i * VEC - plane * nvp.d));
          const BnParam q1 = params[c + 1 == cdiv.d ? 0u : c + 1];
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const bool nx = j >= cross;
            o[j] = (nx ? q1.a : q.a) * dv[u][j] +
                   (nx ? q1.b : q.b) * (xv[u][j] - (nx ? q1.mean : q.mean)) + (nx ? q1.c : q.c);
          }
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = q.a * dv[u][j] + q.b * (xv[u][j] - q.mean) + q.c;
        }
        if (accum) {
          float old[VEC];
          load_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, old);
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] += old[j];
        }
        store_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, o);
      }
    }
  }
}

template <typename T, int VEC, bool FUSED = false>
__global__ void __launch_bounds__(256)
bn_bwd_apply_cl_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                       T *__restrict__ dx, const BnParam *__restrict__ params,
                       uint32_t ncv, uint32_t ntiles, uint32_t M, int accum,
                       const T *__restrict__ y, T *__restrict__ dz, int accum_dz,
                       uint32_t tile_cols) {
  constexpr int U = 2;
  const size_t slab = static_cast<size_t>(blockIdx.y) * M * ncv * VEC;
  x += slab;
  dy += slab;
  if (!FUSED || dx) dx += slab;
  if constexpr (FUSED) {
    y += slab;
    if (dz) dz += slab;
  }
  params += static_cast<size_t>(blockIdx.y) * ncv * VEC;
  const ClApplyMap map = cl_apply_map<U>(ncv, ntiles, tile_cols);
  // dx = pa*dy + pb*(x - mean) + pc = pa*dy + (pb*x + ps), ps = pc - pb*mean:
  // pb*(x-mean) is the small curvature term, so folding the mean costs nothing
  // measurable in float either (|pb*mean| <= |dvar|*2|mean|/N).
  // The coefficients of the block's channels through LDS, a channel per thread
  // (as in the forward kernel: a thread fetching its own VEC parameter structs
  // touches a cache line per lane and load).
  __shared__ float tab[3 * 256 * VEC];
  {
    const uint32_t c0 = (blockIdx.x % ntiles) * tile_cols * VEC;
    const uint32_t nch = min(tile_cols * VEC, ncv * VEC - c0);
    for (uint32_t k = threadIdx.x; k < nch; k += 256u) {
      const BnParam q = params[c0 + k];
      tab[k] = q.a;
      tab[256 * VEC + k] = q.b;
      tab[2 * 256 * VEC + k] = fmaf(-q.b, q.mean, q.c);
    }
    __syncthreads();
  }
  if (!map.active) return;
  const uint32_t cv = map.cv;
  float pa[VEC], pb[VEC], ps[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const uint32_t k = map.col * VEC + j;
    pa[j] = tab[k];
    pb[j] = tab[256 * VEC + k];
    ps[j] = tab[2 * 256 * VEC + k];
  }
  for (uint32_t r0 = map.row0; r0 < M; r0 += map.row_step) {
    RawVec<T, VEC> xr[U], dr[U];
    RawVec<T, VEC> yr[FUSED ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = min(r0 + u * map.R, M - 1) * ncv + cv;
      xr[u] = load_raw<T, VEC>(x + static_cast<size_t>(i) * VEC);
      dr[u] = load_raw<T, VEC>(dy + static_cast<size_t>(i) * VEC);
      if constexpr (FUSED) yr[u] = load_raw<T, VEC>(y + static_cast<size_t>(i) * VEC);
    }
    if constexpr (FUSED) {
#pragma unroll
      for (int u = 0; u < U; ++u) dr[u] = raw_relu_mask<T, VEC>(dr[u], yr[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t row = r0 + u * map.R;
      const uint32_t i = row * ncv + cv;
      if (row < M) {
        if constexpr (FUSED) {
          if (dz) {
            T *dzp = dz + static_cast<size_t>(i) * VEC;
            if (accum_dz) {
              float g[VEC], old[VEC];
              unpack<T, VEC>(dr[u], g);
              load_vec<T, VEC>(dzp, old);
#pragma unroll
              for (int j = 0; j < VEC; ++j) g[j] += old[j];
              store_vec<T, VEC>(dzp, g);
            } else {
              store_raw<T, VEC>(dzp, dr[u]);
            }
          }
          if (!dx) continue;
        }
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          o[j] = elem_fma<T, VEC>(dr[u], j, pa[j], elem_fma<T, VEC>(xr[u], j, pb[j], ps[j]));
        if (accum) {
          float old[VEC];
          load_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, old);
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] += old[j];
        }
        store_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Channel-last Group/InstanceNormalization on the BatchNormalization
// channel-last machinery: x is N slabs [S, C]; the split reductions above
// leave partials per (n, c, split).  The finalize kernels merge the partials
// of each (n, group)'s cpg channels (cpg = 1: InstanceNormalization) and
// publish mean/var of the group plus the apply parameters of its channels.
// WAVE: one wave per (n, group) (small groups, no LDS), else one block.
//   gamma/beta index of channel c in sample n: gmod == 0 ? n*C + c : c
// ---------------------------------------------------------------------------
__device__ __forceinline__ float subgroup_sum(float v, uint32_t width /* power of two <= 64 */) {
  for (uint32_t o = width >> 1; o; o >>= 1) v += __shfl_xor(v, static_cast<int>(o));
  return v;
}

template <bool WAVE>
__global__ void __launch_bounds__(kBnBlock)
gn_cl_finalize_fwd_kernel(const float *__restrict__ part, uint32_t S, uint32_t C, uint32_t cpg,
                          uint32_t NG, float inv_R, float eps, const float *__restrict__ gamma,
                          const float *__restrict__ beta, uint32_t gmod, uint32_t bmod,
                          float *__restrict__ mean, float *__restrict__ var,
                          BnParam *__restrict__ params) {
  __shared__ float lds[3 * (kBnBlock / kWave)];
  constexpr uint32_t kWaves = kBnBlock / kWave;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t ng = WAVE ? blockIdx.x * kWaves + threadIdx.x / kWave : blockIdx.x;
  if (WAVE && ng >= NG) return; // wave-uniform; no block barrier in this mode
  const uint32_t tid = WAVE ? lane : threadIdx.x;
  const uint32_t nthr = WAVE ? kWave : kBnBlock;
  const uint32_t G = C / cpg;
  const uint32_t n = ng / G, g = ng % G;
  const float *p0 = part + 3 * (static_cast<size_t>(n) * C + static_cast<size_t>(g) * cpg) * S;
  Welford w{0.f, 0.f, 0.f};
  for (uint32_t i = tid; i < cpg * S; i += nthr) { // (channel, split) pairs, contiguous
    const float *p = p0 + 3 * static_cast<size_t>(i);
    w = welford_merge(w, Welford{p[0], p[1], p[2]});
  }
  w = WAVE ? wave_welford(w) : block_welford(w, lds);
  const float m = w.mean;
  const float v = w.m2 * inv_R;
  const float istd = inv_std(v, eps);
  if (tid == 0) {
    mean[ng] = m;
    var[ng] = v;
  }
  for (uint32_t cl = tid; cl < cpg; cl += nthr) {
    const uint32_t c = g * cpg + cl;
    const uint32_t nc = n * C + c;
    BnParam q;
    q.mean = m;
    q.a = (gamma ? gamma[gmod ? c : nc] : 1.f) * istd;
    q.b = beta ? beta[bmod ? c : nc] : 0.f;
    q.c = 0.f;
    params[nc] = q;
  }
}

// Backward: per (n, group) s1 = sum_c gamma_c*sdy_c, t2 = sum_c gamma_c*sdx_c
// with sdx_c = sum dy*(x-mean) over the channel (kernel/group_normalization.cuh
// :98-149 on centred sums), then per channel
//   dx = gamma_c*istd*dy + f1*(x-mean) + f2',  f1 = -t2*istd^3/R + 2*dvar/R,
//   f2' = -s1*istd/R + dmean/R
// and the pair (sdx_c*istd, sdy_c) for the batch sum of dgamma/dbeta.
// A wave covers 64/sp channels at a time, sp lanes (a power of two) sharing
// the S splits of one channel.
template <bool WAVE>
__global__ void __launch_bounds__(kBnBlock)
gn_cl_finalize_bwd_kernel(const float *__restrict__ part2, uint32_t S, uint32_t sp, uint32_t C,
                          uint32_t cpg, uint32_t NG, float inv_R, float eps,
                          const float *__restrict__ gamma, uint32_t gmod,
                          const float *__restrict__ mean, const float *__restrict__ var,
                          const float *__restrict__ dmean, const float *__restrict__ dvar,
                          float *__restrict__ pairs, BnParam *__restrict__ params) {
  __shared__ float lds[2 * (kBnBlock / kWave)];
  constexpr uint32_t kWaves = kBnBlock / kWave;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t ng = WAVE ? blockIdx.x * kWaves + wave : blockIdx.x;
  if (WAVE && ng >= NG) return; // wave-uniform; no block barrier in this mode
  const uint32_t tid = WAVE ? lane : threadIdx.x;
  const uint32_t nthr = WAVE ? kWave : kBnBlock;
  const uint32_t G = C / cpg;
  const uint32_t n = ng / G, g = ng % G;
  const float m = mean[ng];
  const float istd = inv_std(var[ng], eps);
  const uint32_t chw = kWave / sp;          // channels per wave pass
  const uint32_t sub = lane / sp, sl = lane & (sp - 1);
  const uint32_t first = (WAVE ? 0u : wave) * chw;
  const uint32_t stride = (WAVE ? 1u : kWaves) * chw;
  const float2 *__restrict__ pp = reinterpret_cast<const float2 *>(part2);
  float s1 = 0.f, t2 = 0.f;
  for (uint32_t cl0 = first; cl0 < cpg; cl0 += stride) {
    const uint32_t cl = cl0 + sub;
    const bool ok = cl < cpg;
    const uint32_t c = g * cpg + (ok ? cl : 0u);
    const uint32_t nc = n * C + c;
    float sdx = 0.f, sdy = 0.f;
    for (uint32_t s = sl; s < S; s += sp) {
      const float2 v = pp[static_cast<size_t>(nc) * S + s];
      sdx += v.x;
      sdy += v.y;
    }
    sdx = subgroup_sum(sdx, sp);
    sdy = subgroup_sum(sdy, sp);
    if (ok && sl == 0) {
      reinterpret_cast<float2 *>(pairs)[nc] = make_float2(sdx * istd, sdy);
      const float gm = gamma ? gamma[gmod ? c : nc] : 1.f;
      s1 += gm * sdy;
      t2 += gm * sdx;
    }
  }
  if (WAVE) {
    s1 = wave_sum(s1);
    t2 = wave_sum(t2);
  } else {
    block_sum2(s1, t2, lds);
  }
  const float f1 = -t2 * istd * istd * istd * inv_R + (dvar ? 2.f * dvar[ng] * inv_R : 0.f);
  const float f2 = -s1 * istd * inv_R + (dmean ? dmean[ng] * inv_R : 0.f);
  for (uint32_t cl = tid; cl < cpg; cl += nthr) {
    const uint32_t c = g * cpg + cl;
    const uint32_t nc = n * C + c;
    BnParam q;
    q.mean = m;
    q.a = (gamma ? gamma[gmod ? c : nc] : 1.f) * istd;
    q.b = f1;
    q.c = f2;
    params[nc] = q;
  }
}

} // namespace nblahip
