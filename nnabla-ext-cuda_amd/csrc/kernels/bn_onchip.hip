// BatchNormalization training with a channel held on one CU: registers first,
// LDS for what exceeds them.  One 1024-thread block per channel reads its N
// planes once, reduces, and writes y: x crosses the memory system once (2 S
// per call) where the split reduction reads it twice (3 S).
//
// A CU holds 512 KB of vector registers and 160 KB of LDS; a 1024-thread block
// may use 128 registers per thread, of which NR 16-byte vectors (4 registers
// each) are data, and NS more vectors per thread live in LDS (each thread
// reads back only what it wrote: no barrier, no bank conflict).  NR + NS = 25
// covers 25600 vectors = 400 KB per channel: [32, C, 56, 56] in float,
// [64, C, 56, 56] in half.  A longer channel keeps that many vectors and
// streams the rest (read twice, as in the split reduction).
//
// The backward keeps x on the CU the same way and streams dy past it twice
// (sums, then dx): x once, dy twice, dx once = 4 S where the split reduction
// moves 5 S; dgamma/dbeta are written by the channel's block, no finalize.
// Beside x a thread needs a batch of dy, so it holds fewer vectors: 18432 per
// channel with 1024 threads, 20480 with 512; the rest of x is streamed with dy
// (its first 3072 vectors parked in the LDS that is left, so that the second
// pass does not read them again).
//
// The block is alone on its CU, so fewer channels than CUs leave CUs idle; the
// path still wins down to an eighth (forward) or a quarter (backward) of the
// CUs, because a CU alone pulls far more than its share of the bandwidth.
//
// The kernels are fully unrolled over the slots of a thread, and most of what
// looks odd below (opaque copies of the thread index, vectors hidden from the
// optimiser, addresses tied to earlier results) keeps the compiler from
// holding across the passes what is cheaper to compute again: each such value
// costs a register in every one of 1024 threads, and the layouts leave none.
#include <algorithm>
#include <type_traits>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"

namespace nblahip {

namespace {

struct BnOnchipArgs {
  const void *x;
  void *y;
  const float *gamma, *beta;
  float *mean, *var, *rmean, *rvar;
  uint32_t C;
  uint32_t size2;      // elements per plane
  uint32_t nv;         // vectors per channel = size0 * vpp
  FastDiv vpp;         // vectors per plane
  float inv_N, unbias, decay, eps, one;
  int vec;       // elements per vector (8-byte vectors for half planes of 4k elements)
  const void *z; // FusedBatchNormalization forward: y = max(0, bn(x) [+ z]); may be null
  // backward
  const void *dy;
  void *dx;                 // may be null
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;    // may be null
  // InstanceNormalization backward through these kernels (a channel = one
  // plane (n, c), C = N*C of them): gamma of channel c % gmod, and the sums
  // go to pairs[c] = (dgamma part, dbeta part) for the batch sum that follows
  uint32_t gmod;
  float *pairs; // may be null
  int accum_dx, accum_g, accum_b;
  // Planes that are no whole number of 128-byte lines share their first and
  // last line with the neighbouring channels' planes: plane_bytes != 0 then,
  // and neighbouring channels run on the same XCD (per_xcd channels each).
  uint32_t plane_bytes;
  uint32_t per_xcd;
};

// Channel of block b.  Workgroups go to the 8 XCDs round-robin by index; with
// planes that share lines, neighbouring channels take the same XCD, whose L2
// then fetches a shared line once and merges the partial writes to it.
__device__ __forceinline__ uint32_t onchip_channel(const BnOnchipArgs &a, uint32_t b) {
  return a.per_xcd ? (b % 8u) * a.per_xcd + b / 8u : b;
}

// Writes vector v of the channel (at dst).  A vector in a line that the plane
// shares with a neighbour is written with an ordinary store, which L2 merges
// with the neighbour's part of the line; non-temporal stores of line pieces
// go to memory piece by piece.
template <typename T, int VEC>
__device__ __forceinline__ void onchip_store(const BnOnchipArgs &a, T *dst, uint32_t v,
                                             const float (&o)[VEC]) {
  if (a.plane_bytes) {
    const uint32_t w = v - a.vpp.div(v) * a.vpp.d;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
    const uintptr_t first = addr - static_cast<uintptr_t>(w) * sizeof(RawVec<T, VEC>);
    const uintptr_t line = addr >> 7;
    if (line < ((first + 127u) >> 7) || line >= ((first + a.plane_bytes) >> 7)) {
      store_vec<T, VEC, false>(dst, o);
      return;
    }
  }
  store_vec<T, VEC>(dst, o);
}

// Element offset of vector v of channel c (planes are contiguous, a channel's
// planes lie C*size2 apart).
__device__ __forceinline__ uint32_t onchip_offset(const BnOnchipArgs &a, uint32_t c, uint32_t v,
                                                  int vec) {
  const uint32_t n = a.vpp.div(v);
  const uint32_t w = v - n * a.vpp.d;
  return (n * a.C + c) * a.size2 + w * static_cast<uint32_t>(vec);
}

} // namespace

// OVER: the channel is longer than the NR + NS slots held on chip.  The rest
// is read once for the statistics (into the same per-thread sums as the held
// part) and a second time for y: 2 S + (1 - 25600 / nv) S instead of 3 S.
// FUSED (FusedBatchNormalization): y = max(0, bn(x) + z), z optional.
template <typename T, int VEC, int NR, int NS, bool OVER = false, bool FUSED = false>
__global__ void __launch_bounds__(kOnchipBlock)
bn_onchip_fwd_kernel(const BnOnchipArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == sizeof(Slot<T, VEC>), "8- or 16-byte vectors");
  __shared__ float red[kOnchipBlock / kWave];
  __shared__ Slot<T, VEC> spill[NS > 0 ? NS * kOnchipBlock : 1];
  const uint32_t c = onchip_channel(a, blockIdx.x);
  const uint32_t t = threadIdx.x;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.y);
  // (asked for now: behind the block sums they would cost a round trip of their own)
  const float gamma_c = a.gamma ? a.gamma[c] : 1.f;
  const float beta_c = a.beta ? a.beta[c] : 0.f;

  // Loads, all in flight together (no branch: a slot beyond the channel reads
  // the channel's last vector and is left out of every sum and store): the LDS
  // part first (its registers are handed back as soon as the values are
  // parked), then the register part.
  RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t;
    parked[k] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
  }
  RawVec<T, VEC> raw[NR];
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
    raw[k] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
  }
  // Statistics from sums every wave takes over its OWN registers as its loads
  // arrive (the memory system serves a CU's waves one after the other: what a
  // wave does before the block's first barrier hides behind the other waves'
  // loads, a second pass about the block's mean would keep memory idle).  Per
  // thread: s = sum x, then about the thread's own mean K = s / n:
  // s1 = sum (x - K) (rounding residue), s2 = sum (x - K)^2; mean = sum_t s / N
  // and, about it, var = sum_t (s2 + 2 e s1 + n e^2) / N with e = K - mean: two
  // block sums of a few operations per thread.  sum_t n e^2 is the variance
  // between the threads' means, never more than the total: nothing cancels,
  // whatever the data.
  // (OVER: the vectors beyond the held ones are read here once, shifted by the
  // K of the thread's held elements, and once more for y.)
  auto held = [&](int k) { return static_cast<int>(t) < static_cast<int>(a.nv) - k * kOnchipBlock; };
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const float part = raw_sum<T, VEC>(parked[k], 0.f);
    s += held(NR + k) ? part : 0.f;
    spill[k * kOnchipBlock + t] = __builtin_bit_cast(Slot<T, VEC>, parked[k]);
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const float part = raw_sum<T, VEC>(raw[k], 0.f);
    s += held(k) ? part : 0.f;
  }
  constexpr uint32_t kHeld = static_cast<uint32_t>(NR + NS) * kOnchipBlock;
  const uint32_t nvh = OVER ? min(a.nv, kHeld) : a.nv; // held vectors of the channel
  const float nh = t < nvh ? static_cast<float>(((nvh - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
  const float kk = s * (1.0f / fmaxf(nh, 1.f));
  float s1 = 0.f, s2 = 0.f;
  auto take = [&](const RawVec<T, VEC> &r) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = elem_fma<T, VEC>(r, j, a.one, -kk);
      s1 += d;
      s2 = fmaf(d, d, s2);
    }
  };
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    if (held(NR + k)) take(parked[k]);
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    if (held(k)) take(raw[k]);
  }
  float nt = nh; // elements of the thread, held and streamed
  if constexpr (OVER) {
    constexpr int BO = 4;
#pragma unroll 1
    for (uint32_t v0 = kHeld; v0 < a.nv; v0 += BO * kOnchipBlock) {
      RawVec<T, VEC> xo[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b)
        xo[b] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v0 + b * kOnchipBlock + t, a.nv - 1u), VEC));
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        if (v0 + b * kOnchipBlock + t < a.nv) take(xo[b]);
      }
    }
    nt = t < a.nv ? static_cast<float>(((a.nv - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
  }
  // (n K + s1 = the thread's sum of x, held and streamed)
  const float mean = onchip_block_sum(fmaf(nt, kk, s1), red) * a.inv_N;
  const float e = kk - mean;
  const float var = onchip_block_sum(fmaf(e, fmaf(nt, e, 2.f * s1), s2), red) * a.inv_N;
#pragma unroll
  for (int k = 0; k < NR; ++k) keep_packed<T, VEC>(raw[k]);
  const float istd = inv_std(var, a.eps);
  if (t == 0) {
    a.mean[c] = mean;
    a.var[c] = var;
    if (a.rmean) a.rmean[c] = a.decay * a.rmean[c] + (1.f - a.decay) * mean;
    if (a.rvar) a.rvar[c] = a.decay * a.rvar[c] + (1.f - a.decay) * var * a.unbias;
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) keep_packed<T, VEC>(raw[k]);
  const float g = gamma_c * istd;
  const float b = beta_c;
  const float sh = fmaf(-mean, g, b);

  auto emit = [&](const RawVec<T, VEC> &r, uint32_t v) {
    float o[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      if constexpr (sizeof(T) == 2) {
        o[j] = elem_fma<T, VEC>(r, j, g, sh); // x*g + (b - mean*g): one mixed fma, rounded once
      } else {
        o[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mean), g, b);
      }
    }
    const uint32_t off = onchip_offset(a, c, v, VEC);
    if constexpr (FUSED) {
      if (a.z) {
        const RawVec<T, VEC> zr = load_raw<T, VEC>(static_cast<const T *>(a.z) + off);
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = elem_fma<T, VEC>(zr, j, a.one, o[j]);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = fmaxf(0.f, o[j]);
    }
    onchip_store<T, VEC>(a, y + off, v, o);
  };
  const uint32_t t2 = fresh(t);
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
    if (v < a.nv) emit(raw[k], v);
  }
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t2;
    if (v < a.nv) emit(__builtin_bit_cast(RawVec<T, VEC>, spill[k * kOnchipBlock + t]), v);
  }
  if constexpr (OVER) {
    constexpr int BO = 4;
#pragma unroll 1
    for (uint32_t v0 = kHeld; v0 < a.nv; v0 += BO * kOnchipBlock) {
      RawVec<T, VEC> xo[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b)
        xo[b] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v0 + b * kOnchipBlock + t, a.nv - 1u), VEC));
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        const uint32_t v = v0 + b * kOnchipBlock + t;
        if (v < a.nv) emit(xo[b], v);
      }
    }
  }
}


// Backward (batch statistics).  mean/var are read; with xh = (x-mean)*istd:
//   sdy = sum dy, sdx = sum dy*xh  (= dbeta, dgamma)
//   dx = dy*g*istd + xh*cA + cb,  cA = -istd*g*sdx/N + 2*dvar*std/N,
//   cb = -g*sdy*istd/N + dmean/N.
// dy is streamed in batches of B vectors per thread, twice.
// TB threads per block: a CU's 512 KB of registers are 128 per thread for 1024
// threads and 256 for 512, and what a thread needs beside its data (addresses,
// sums, a batch of dy) is paid once per thread - the long channels take 512
// threads (and 320 bytes of LDS per thread instead of 160).
// OVER: the channel is longer than the NR + NS slots held on chip; the
// vectors beyond them are streamed like dy (x and dy read in both passes, a
// rolled loop of small batches), so only the held part - and what the first
// pass parks in LDS - saves its second read: (21504 / nv) S of the 5 S.
template <typename T, int VEC, int NR, int NS, int B, int TB, bool OVER = false>
__global__ void __launch_bounds__(TB)
bn_onchip_bwd_kernel(const BnOnchipArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == sizeof(Slot<T, VEC>), "8- or 16-byte vectors");
  constexpr int NL = NR + NS;
  // OVER: the LDS the held slots leave free parks the first NX slots of x
  // beyond them on their way through the first pass (each thread reads back
  // only what it wrote), so the second pass reads those from LDS, not again
  // from memory: (5 - (NL + NX) * TB / nv) S.
  constexpr int NX = (OVER && TB == 1024) ? (9 - NS > 0 ? 9 - NS : 0) : 0;
  __shared__ float red[TB / kWave];
  __shared__ Slot<T, VEC> spill[NS > 0 ? NS * TB : 1];
  __shared__ Slot<T, VEC> extra[NX > 0 ? NX * TB : 1];
  const uint32_t c = onchip_channel(a, blockIdx.x);
  const uint32_t t = threadIdx.x;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.dx);
  // (asked for now: behind the block sums they would cost a round trip of their own)
  const float g = a.gamma ? a.gamma[c % a.gmod] : 1.f;

  RawVec<T, VEC> raw[NR];
  {
    RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const uint32_t v = static_cast<uint32_t>(NR + k) * TB + t;
      parked[k] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
    }
    // Here the parked vectors are stored away before the register part is
    // requested (its addresses wait for the last parked value): with all 25
    // loads in flight plus the first batch of dy the kernel spills.
    uint32_t tr = t;
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const Slot<T, VEC> w = __builtin_bit_cast(Slot<T, VEC>, parked[k]);
      spill[k * TB + t] = w;
      tr = fresh_after(tr, w.x);
    }
    __builtin_amdgcn_sched_barrier(0); // every LDS store above, every load of the register part below
    // The parked values must be read back from LDS, not forwarded from the
    // registers that held them (which would keep those registers alive).
    asm volatile("" ::: "memory");
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const uint32_t v = static_cast<uint32_t>(k) * TB + tr;
      raw[k] = load_raw<T, VEC>(x + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
    }
  }
  const float mean = a.mean[c];
  const float vpe = a.var[c] + a.eps;
  const float istd = 1.0f / sqrtf(vpe);
  const float nmi = -mean * istd;

  // (k is a compile-time constant after unrolling; tid is the batch's own
  // copy of the thread index, so that the LDS reads of a batch are not issued
  // before the batch before it is done)
  auto xvec = [&](int k, uint32_t tid) -> RawVec<T, VEC> {
    if (k < NR) return raw[k < NR ? k : 0];
    return __builtin_bit_cast(RawVec<T, VEC>, spill[(k - NR) * TB + tid]);
  };

  float sdy = 0.f, sdx = 0.f;
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t t1 = fresh_after(t, sdx);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int k = k0 + b;
      d[b] = zero_raw<T, VEC>();
      if (k < NL) { // compile-time
        const uint32_t v = static_cast<uint32_t>(k) * TB + t1;
        d[b] = load_raw<T, VEC>(dy + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int k = k0 + b;
      if (k < NL) {
        const RawVec<T, VEC> xr = xvec(k, t1);
        float py = raw_sum<T, VEC>(d[b], 0.f), px = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr, j, mean, istd, nmi);
          px = elem_fma<T, VEC>(d[b], j, xh, px);
        }
        const bool ok = static_cast<int>(t) < static_cast<int>(a.nv) - k * TB; // t against a scalar
        sdy += ok ? py : 0.f;
        sdx += ok ? px : 0.f;
      }
    }
    // keep the next batch's loads below this point: hoisted, the batches'
    // registers add up and spill
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (OVER) {
    constexpr int BO = 2;
#pragma unroll 1
    for (uint32_t v0 = static_cast<uint32_t>(NL) * TB; v0 < a.nv; v0 += BO * TB) {
      RawVec<T, VEC> xo[BO], d[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        const uint32_t off = onchip_offset(a, c, min(v0 + b * TB + t, a.nv - 1u), VEC);
        xo[b] = load_raw<T, VEC>(x + off);
        d[b] = load_raw<T, VEC>(dy + off);
      }
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        if constexpr (NX > 0) {
          // (the slot index is the same for the whole block: a scalar branch)
          const uint32_t slot = (v0 - static_cast<uint32_t>(NL) * TB) / TB + b;
          if (slot < static_cast<uint32_t>(NX)) extra[slot * TB + t] = __builtin_bit_cast(Slot<T, VEC>, xo[b]);
        }
        float py = raw_sum<T, VEC>(d[b], 0.f), px = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xo[b], j, mean, istd, nmi);
          px = elem_fma<T, VEC>(d[b], j, xh, px);
        }
        const bool ok = v0 + b * TB + t < a.nv;
        sdy += ok ? py : 0.f;
        sdx += ok ? px : 0.f;
      }
    }
  }
  sdy = onchip_block_sum<TB>(sdy, red);
  sdx = onchip_block_sum<TB>(sdx, red);
  if (t == 0) {
    if (a.dgamma) a.dgamma[c] = sdx + (a.accum_g ? a.dgamma[c] : 0.f);
    if (a.dbeta) a.dbeta[c] = sdy + (a.accum_b ? a.dbeta[c] : 0.f);
    if (a.pairs) {
      a.pairs[2 * c] = sdx;
      a.pairs[2 * c + 1] = sdy;
    }
  }
  if (dx == nullptr) return;
#pragma unroll
  for (int k = 0; k < NR; ++k) forget<T, VEC>(raw[k]);
  const float gi = g * istd;
  const float cA = -istd * g * sdx * a.inv_N + (a.dvar ? 2.f * a.dvar[c] * (vpe * istd) * a.inv_N : 0.f);
  const float cb = -g * sdy * istd * a.inv_N + (a.dmean ? a.dmean[c] * a.inv_N : 0.f);
  float last = cb; // something the previous batch computed
#pragma unroll
  for (int k0 = 0; k0 < NL; k0 += B) {
    const uint32_t t2 = fresh_after(t, last);
    RawVec<T, VEC> d[B];
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int k = k0 + b;
      d[b] = zero_raw<T, VEC>();
      if (k < NL) { // compile-time
        const uint32_t v = static_cast<uint32_t>(k) * TB + t2;
        d[b] = load_raw<T, VEC>(dy + onchip_offset(a, c, min(v, a.nv - 1u), VEC));
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int k = k0 + b;
      const uint32_t v = static_cast<uint32_t>(k) * TB + t2;
      if (k < NL && v < a.nv) {
        const RawVec<T, VEC> xr = xvec(k, t2);
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr, j, mean, istd, nmi);
          o[j] = elem_fma<T, VEC>(d[b], j, gi, fmaf(xh, cA, cb));
        }
        T *dst = dx + onchip_offset(a, c, v, VEC);
        if (a.accum_dx) {
          float old[VEC];
          load_vec<T, VEC>(dst, old);
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] += old[j];
        }
        onchip_store<T, VEC>(a, dst, v, o);
        last = o[0];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (OVER) {
    constexpr int BO = 2;
#pragma unroll 1
    for (uint32_t v0 = static_cast<uint32_t>(NL) * TB; v0 < a.nv; v0 += BO * TB) {
      RawVec<T, VEC> xo[BO], d[BO];
      uint32_t off[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        off[b] = onchip_offset(a, c, min(v0 + b * TB + t, a.nv - 1u), VEC);
        bool parked = false;
        if constexpr (NX > 0) {
          const uint32_t slot = (v0 - static_cast<uint32_t>(NL) * TB) / TB + b;
          parked = slot < static_cast<uint32_t>(NX);
          if (parked) xo[b] = __builtin_bit_cast(RawVec<T, VEC>, extra[slot * TB + t]);
        }
        if (!parked) xo[b] = load_raw<T, VEC>(x + off[b]);
        d[b] = load_raw<T, VEC>(dy + off[b]);
      }
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        if (v0 + b * TB + t < a.nv) {
          float o[VEC];
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float xh = norm_elem<T, VEC>(xo[b], j, mean, istd, nmi);
            o[j] = elem_fma<T, VEC>(d[b], j, gi, fmaf(xh, cA, cb));
          }
          T *dst = dx + off[b];
          if (a.accum_dx) {
            float old[VEC];
            load_vec<T, VEC>(dst, old);
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] += old[j];
          }
          onchip_store<T, VEC>(a, dst, v0 + b * TB + t, o);
        }
      }
    }
  }
}

namespace {

template <typename T, int VEC, bool FUSED>
int run_onchip_fwd(int nl, const BnOnchipArgs &a, hipStream_t st) {
#define ONCHIP_CASE(NR, NS)                                                                      \
  if (nl <= (NR) + (NS)) {                                                                       \
    NBLAHIP_LAUNCH(FUSED ? "bn_onchip_fwd_kernel_fused" : "bn_onchip_fwd_kernel",                \
                   (bn_onchip_fwd_kernel<T, VEC, NR, NS, false, FUSED>), dim3(a.C),              \
                   dim3(kOnchipBlock), 0, st, a);                                                \
    return last_launch_status();                                                                 \
  }
  ONCHIP_CASE(10, 0)
  ONCHIP_CASE(12, 0)
  ONCHIP_CASE(14, 0)
  ONCHIP_CASE(16, 0)
  ONCHIP_CASE(16, 3)
  ONCHIP_CASE(16, 6)
  ONCHIP_CASE(16, 9)
#undef ONCHIP_CASE
  // longer channels: 25 slots held, the rest streamed
  NBLAHIP_LAUNCH(FUSED ? "bn_onchip_fwd_kernel_fused" : "bn_onchip_fwd_kernel",
                 (bn_onchip_fwd_kernel<T, VEC, 16, 9, true, FUSED>), dim3(a.C), dim3(kOnchipBlock),
                 0, st, a);
  return last_launch_status();
}

template <typename T, int VEC>
int run_onchip_bwd(int64_t nv, const BnOnchipArgs &a, hipStream_t st) {
#define ONCHIP_CASE(NR, NS, B, TB)                                                               \
  if (nv <= static_cast<int64_t>((NR) + (NS)) * (TB)) {                                          \
    NBLAHIP_LAUNCH("bn_onchip_bwd_kernel", (bn_onchip_bwd_kernel<T, VEC, NR, NS, B, TB>),        \
                   dim3(a.C), dim3(TB), 0, st, a);                                               \
    return last_launch_status();                                                                 \
  }
  ONCHIP_CASE(10, 0, 4, 1024)
  ONCHIP_CASE(12, 0, 4, 1024)
  ONCHIP_CASE(14, 0, 4, 1024)
  ONCHIP_CASE(12, 3, 4, 1024)
  ONCHIP_CASE(12, 6, 4, 1024)
  ONCHIP_CASE(24, 16, 8, 512)
#undef ONCHIP_CASE
  // longer channels: 18 slots held, the rest streamed
  NBLAHIP_LAUNCH("bn_onchip_bwd_kernel", (bn_onchip_bwd_kernel<T, VEC, 12, 6, 4, 1024, true>),
                 dim3(a.C), dim3(1024), 0, st, a);
  return last_launch_status();
}

// Planes that share lines with their neighbours: edge stores and the XCD map.
void onchip_edge_plan(BnOnchipArgs &a, int64_t plane_bytes) {
  a.plane_bytes = 0;
  a.per_xcd = 0;
  // Short planes only, where two of a handful of lines are shared: 784-byte
  // planes ([256,1024,14,14] float) forward 106.3 -> 94.9 us, [256,256,14,14]
  // 25.4 / 34.4 -> 20.3 / 31.1 us, 392-byte planes ([256,1024,14,14] half)
  // forward 54.9 -> 43.3 us; with 1568-byte planes ([256,512,28,28] half) the
  // forward gains 2 % and the backward, which reads dy twice through the same
  // L2, loses 4 %.
  if (plane_bytes % 128 == 0 || plane_bytes > tune_int("BN_EDGE_STORES_MAX_BYTES", 1024)) return;
  a.plane_bytes = static_cast<uint32_t>(plane_bytes);
  if (a.C % 8 == 0) a.per_xcd = a.C / 8;
}

// Shape test shared by both directions; fills the common arguments.
bool onchip_args(const BnProblem &p, bool backward, BnOnchipArgs &a, int &nl, int max_nl = 25) {
  if (!tune_int("BN_ONCHIP", 1)) return false;
  if (p.size2 <= 1 || p.y || p.dz || p.sums_out || p.sums_in) return false;
  if (backward && (p.relu || p.z)) return false;
  if (p.z && !aligned16(p.z)) return false;
  int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.dtype == NBLAHIP_F16 && p.size2 % 8 != 0 && p.size2 % 4 == 0) vec = 4; // 8-byte vectors
  if (p.size2 % vec != 0 || !aligned16(p.x) || (p.out && !aligned16(p.out))) return false;
  if (backward && !aligned16(p.dy)) return false;
  const int64_t nv = p.size0 * (p.size2 / vec);
  nl = static_cast<int>((nv + kOnchipBlock - 1) / kOnchipBlock);
  // up to 8 loads per thread the row kernels take the channel; above 25 it
  // does not fit
  if (nl <= 8 || nl > max_nl) return false;
  // 8-byte vectors move half as much per instruction: a gain for channels of
  // up to 16384 of them ([256,1024,14,14] 61 / 84 -> 58 / 77 us, [256,256,14,14]
  // 24 / 24.5 -> 15 / 18.5 us), a loss beyond ([512,1024,14,14] 115 / 175 -> 130 / 176 us)
  if (vec == 4 && p.dtype == NBLAHIP_F16 && nl > 16) return false;
  // A block is alone on its CU, so fewer channels than CUs leave CUs idle -
  // but a CU alone pulls far more than its 1/256 share of the bandwidth, and
  // the split reduction pays two launches more per direction: with whole
  // channels held, both directions win at every channel count (kernel time of
  // forward + backward, [16,C,56,56] float: 18.1 vs 26.7 us at C = 8, 19.4 vs
  // 21.1 at 32, 24.2 vs 25.9 at 60; [32,C,56,56] half: 22.5 vs 26.7 at C = 4,
  // 23.4 vs 28.3 at 28).  With a streamed remainder (channels beyond what the
  // layouts hold) from channels for 37 % of the CUs: [32,C,56,56] float forward +
  // backward 39.3 vs 31.8 us at C = 32, 42.0 vs 38.7 at 64, 43.8 vs 44.6 at 80,
  // 46.7 vs 50.6 at 96, 55.1 vs 63.5 at 128, 88.4 vs 99.3 at 224; [32,C,112,112]
  // half 105.6 vs 75.9 at 64, 113.9 vs 112.5 at 96, 124.3 vs 126.9 at 112, 119.5
  // vs 140.1 at 128.  (Only where no channel split over several blocks applies:
  // that takes these shapes first, 24 - 42 us on the float ones.)
  const bool whole = nv <= (backward ? 20480 : 25600);
  const int min_pct = !whole     ? tune_int("BN_ONCHIP_STREAMED_MIN_PCT", 37)
                      : backward ? tune_int("BN_ONCHIP_BWD_MIN_PCT", 1)
                                 : tune_int("BN_ONCHIP_FWD_MIN_PCT", 1);
  if (p.C * 100 < static_cast<int64_t>(device_cus()) * min_pct) return false;
  a = BnOnchipArgs{};
  a.x = p.x;
  a.gamma = p.gamma;
  a.C = static_cast<uint32_t>(p.C);
  a.size2 = static_cast<uint32_t>(p.size2);
  a.nv = static_cast<uint32_t>(nv);
  a.vpp = FastDiv(static_cast<uint32_t>(p.size2 / vec));
  a.vec = vec;
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  a.inv_N = static_cast<float>(1.0 / N);
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  a.gmod = a.C;
  onchip_edge_plan(a, p.size2 * (p.dtype == NBLAHIP_F16 ? 2 : 4));
  return true;
}

} // namespace

bool bn_onchip_bwd(const BnProblem &p, hipStream_t st, int *status) {
  BnOnchipArgs a;
  int nl = 0;
  if (!p.batch_stat || (!p.out && !p.dgamma && !p.dbeta)) return false;
  // Beside x a thread holds a batch of dy: layouts that hold more than 20480
  // vectors per channel spill and lose to the split reduction (25088 vectors,
  // float [32,256,56,56]: 72-76 vs 71 us; half [64,256,56,56]: 115 vs 71 us).
  // Longer channels keep 18432 vectors on chip and stream the rest.
  if (!onchip_args(p, true, a, nl, tune_int("BN_ONCHIP_BWD_MAX", 64))) return false;
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
  *status = p.dtype != NBLAHIP_F16 ? run_onchip_bwd<float, 4>(a.nv, a, st)
            : a.vec == 8           ? run_onchip_bwd<__half, 8>(a.nv, a, st)
                                   : run_onchip_bwd<__half, 4>(a.nv, a, st);
  return true;
}

// InstanceNormalization backward for planes beyond what a block's registers
// hold of x and dy together: x of a plane stays on its CU while dy is streamed
// past it twice (4 S; the streaming kernels move 5 S).  Planes of 8193..20480
// full vectors, at least a quarter as many as there are CUs; up to 65536 with
// the first 18432 held.  The per-plane
// sums are left in p.ws for the batch sum (or the split) that follows.
bool in_onchip_bwd(const RowProblem &p, hipStream_t st, int *status) {
  if (!tune_int("ROW_ONCHIP", 1) || p.mode != kRowIN) return false;
  if (!p.out && !p.dgamma && !p.dbeta) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.R % vec != 0 || !aligned16(p.x) || !aligned16(p.dy) || (p.out && !aligned16(p.out)))
    return false;
  const int64_t nv = p.R / vec;
  if (nv <= 8192 || nv > 65536) return false;
  // (whole planes: from any number of them - [1,C,256,256] float forward +
  // backward 30.8 vs 36.6 us of kernel time at C = 32, 35.0 vs 42.6 at 56;
  // longer planes keep 18432 vectors and stream the rest, which pays only with
  // a plane for nearly every CU: [1,C,512,512] float 123 vs 67 us at C = 32,
  // 135 vs 99 at 56)
  const int min_pct = nv <= 20480 ? tune_int("ROW_ONCHIP_BWD_MIN_PCT", 1)
                                  : tune_int("ROW_ONCHIP_STREAMED_MIN_PCT", 88);
  if (p.rows * 100 < static_cast<int64_t>(device_cus()) * min_pct) return false;
  BnOnchipArgs a{};
  a.x = p.x;
  a.dy = p.dy;
  a.dx = p.out;
  a.gamma = p.gamma;
  a.gmod = static_cast<uint32_t>(p.bc_gamma ? p.channels : p.rows);
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.pairs = (p.dgamma || p.dbeta) ? static_cast<float *>(p.ws) : nullptr;
  a.accum_dx = p.accum_dx;
  a.C = static_cast<uint32_t>(p.rows);
  a.size2 = static_cast<uint32_t>(p.R);
  a.nv = static_cast<uint32_t>(nv);
  a.vpp = FastDiv(static_cast<uint32_t>(nv)); // one plane per channel
  a.vec = vec;
  a.inv_N = static_cast<float>(1.0 / static_cast<double>(p.R));
  a.eps = p.eps;
  a.one = 1.0f;
  onchip_edge_plan(a, p.R * (p.dtype == NBLAHIP_F16 ? 2 : 4));
  *status = p.dtype != NBLAHIP_F16 ? run_onchip_bwd<float, 4>(nv, a, st)
                                   : run_onchip_bwd<__half, 8>(nv, a, st);
  return true;
}

bool bn_onchip_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnOnchipArgs a;
  int nl = 0;
  if (!p.out || !onchip_args(p, false, a, nl, tune_int("BN_ONCHIP_FWD_MAX", 64))) return false;
  a.y = p.out;
  a.beta = p.beta;
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  a.z = p.z;
  if (p.relu || p.z) {
    *status = p.dtype != NBLAHIP_F16 ? run_onchip_fwd<float, 4, true>(nl, a, st)
              : a.vec == 8           ? run_onchip_fwd<__half, 8, true>(nl, a, st)
                                     : run_onchip_fwd<__half, 4, true>(nl, a, st);
  } else {
    *status = p.dtype != NBLAHIP_F16 ? run_onchip_fwd<float, 4, false>(nl, a, st)
              : a.vec == 8           ? run_onchip_fwd<__half, 8, false>(nl, a, st)
                                     : run_onchip_fwd<__half, 4, false>(nl, a, st);
  }
  return true;
}

} // namespace nblahip
