// InstanceNormalization over planes that are no whole number of 16-byte vectors
// (63 x 63, 65 x 65, 7 x 9 ...), register-cached, with 16-byte loads all the same.
//
// A row (one plane of one sample and channel, R elements) then starts anywhere
// inside a vector.  The threads of a row take the TENSOR's aligned vectors that
// meet the row - the first and the last are shared with the neighbouring rows -
// zero the elements outside the row as they arrive, and store the shared
// vectors element by element (the neighbours' elements belong to other waves).
// Everything else is the plain row kernel: the row stays in registers between
// the statistics and the normalization (2 S forward, 3 S backward), one row per
// TPR threads, several rows per block for short rows.  With scalar loads
// instead these planes ran at 2 - 4 copies' time.
//
// The tensor may end inside the last vector of its last row: that one vector is
// loaded element by element.
//
// GroupNormalization whose planes are no whole number of vectors takes the same
// route (gn_masked_*): a row is a group's planes, a vector may hold the end of
// one channel and the start of the next, so gamma / beta are picked per element
// (one boundary per vector at most: planes of VEC elements and more) and the
// backward's per-channel sums are split at that boundary.  Where a group's
// planes fit a block side by side (gn_planes_masked_*), every plane has threads
// of its own and the planes meet only in the sums.
//
// BatchNormalization in the planes layout (bn_masked_*): a block holds its
// channel, the N planes (n, c), through the same pieces.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"
#include "rows.cuh"
#include "rows_dispatch.hpp"

namespace nblahip {

namespace {

struct MaskedRowArgs {
  const void *x;
  const void *dy; // backward only
  void *out;      // y (forward) or dx (backward, may be null)
  const float *gamma, *beta;
  float *mean, *var;
  const float *dmean, *dvar; // may be null
  float *ws;                 // backward: (sum dy*xh, sum dy) per row
  int rows;
  int R;
  long long total; // elements of the tensor = rows * R
  uint32_t pmod, pmod_b; // parameter index = row % pmod (beta: pmod_b)
  float eps, inv_R, one;
  int accum_dx;
  // GroupNormalization: elements per plane, channels per group (pmod = groups;
  // parameter index = (row % pmod) * cpg + element / plane)
  FastDiv plane;
  uint32_t cpg;
};

// The part of the row that vector v of the row's threads holds.
struct RowPiece {
  int col;   // the vector's first element, relative to the row's first (negative: before the row)
  int lo, hi; // elements [lo, hi) of the vector belong to the row
  bool ok;   // the vector meets the row
  bool tail; // the tensor ends inside the vector
};

template <int VEC>
__device__ __forceinline__ RowPiece row_piece(const MaskedRowArgs &a, size_t base, int head, int v) {
  RowPiece p;
  p.col = v * VEC - head;
  p.ok = p.col < a.R; // (head < VEC and v >= 0: the vector never ends before the row)
  p.lo = p.col < 0 ? -p.col : 0;
  p.hi = min(VEC, a.R - p.col);
  p.tail = static_cast<long long>(base) + p.col + VEC > a.total;
  return p;
}

// Elements [lo, hi) of the vector at src, one load each, zeros elsewhere.
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> load_elements(const T *src, int lo, int hi) {
  RawVec<T, VEC> r;
  auto in = [&](int j) { return j >= lo && j < hi; };
  if constexpr (sizeof(T) == 4) {
    static_assert(VEC == 4, "float vectors are 4 wide");
    r.v.x = in(0) ? src[0] : 0.f;
    r.v.y = in(1) ? src[1] : 0.f;
    r.v.z = in(2) ? src[2] : 0.f;
    r.v.w = in(3) ? src[3] : 0.f;
  } else {
    static_assert(VEC == 8, "half vectors are 8 wide");
    const unsigned short *h = reinterpret_cast<const unsigned short *>(src);
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t a0 = in(2 * i) ? h[2 * i] : 0u;
      const uint32_t a1 = in(2 * i + 1) ? h[2 * i + 1] : 0u;
      w[i] = a0 | (a1 << 16);
    }
    r.v = make_uint4(w[0], w[1], w[2], w[3]);
  }
  return r;
}

// The piece's vector with the elements outside the row zeroed (all of it when
// the vector does not meet the row; the load itself is unconditional, from the
// row's first vector then).
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> load_piece(const T *row, int head, const RowPiece &p) {
  const T *src = row + (p.ok ? p.col : -head);
  RawVec<T, VEC> r;
  if (p.ok && p.tail) return load_elements<T, VEC>(src, p.lo, p.hi);
  r = raw_or_zero<T, VEC>(p.ok, load_raw<T, VEC>(src));
  if (p.lo > 0 || p.hi < VEC) r = raw_keep_range<T, VEC>(r, p.lo, p.hi);
  return r;
}

// o[] to the piece: a whole vector, or its elements inside the row.
template <typename T, int VEC>
__device__ __forceinline__ void store_piece(T *row, const RowPiece &p, const float (&o)[VEC], int accum) {
  T *dst = row + p.col;
  if (p.lo == 0 && p.hi == VEC) {
    float out[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[j] = o[j];
    if (accum) {
      float old[VEC];
      load_vec<T, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) out[j] += old[j];
    }
    store_vec<T, VEC>(dst, out);
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      if (j >= p.lo && j < p.hi) dst[j] = from_f32<T>(o[j] + (accum ? to_f32<T>(dst[j]) : 0.f));
    }
  }
}

} // namespace

template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(RowBlock<TPR>::kBlock)
in_masked_fwd_kernel(const MaskedRowArgs a) {
  constexpr int RPB = RowBlock<TPR>::kRowsPerBlock;
  __shared__ float lds[2 * 16];
  const int t = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x) * RPB + sub; row < a.rows; row += gridDim.x * RPB) {
    const size_t base = static_cast<size_t>(row) * a.R;
    const int head = static_cast<int>(base % VEC);
    // (asked for ahead of the row: behind the reductions they would cost a round trip)
    const float g = a.gamma ? a.gamma[static_cast<uint32_t>(row) % a.pmod] : 1.f;
    const float b = a.beta ? a.beta[static_cast<uint32_t>(row) % a.pmod_b] : 0.f;
    RawVec<T, VEC> raw[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k)
      raw[k] = load_piece<T, VEC>(x + base, head, row_piece<VEC>(a, base, head, k * TPR + t));
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
    const float mean = row_sum<TPR>(s, lds) * a.inv_R;
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
          q = (j >= p.lo && j < p.hi) ? fmaf(d, d, q) : q;
        }
      }
    }
    const float var = row_sum<TPR>(q, lds) * a.inv_R;
    const float istd = inv_std(var, a.eps);
    if (t == 0) {
      a.mean[row] = mean;
      a.var[row] = var;
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    const float gs = g * istd;
    const float sh = fmaf(-mean, gs, b);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if constexpr (sizeof(T) == 2) {
            o[j] = elem_fma<T, VEC>(raw[k], j, gs, sh);
          } else {
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), gs, b);
          }
        }
        store_piece<T, VEC>(y + base, p, o, 0);
      }
    }
  }
}

// Backward.  With xh = (x - mean) * istd: sdx = sum dy*xh, sdy = sum dy (the
// row's share of dgamma / dbeta, written to ws[row]), and
//   dx = dy*g*istd + xh*cA + cb,  cA = -istd*g*sdx/R + 2*dvar*std/R,
//   cb = -g*sdy*istd/R + dmean/R.
// Elements outside the row hold dy = 0 (and x = 0), which keeps them out of
// both sums.
template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(RowBlock<TPR>::kBlock)
in_masked_bwd_kernel(const MaskedRowArgs a) {
  constexpr int RPB = RowBlock<TPR>::kRowsPerBlock;
  __shared__ float lds[2 * 16];
  const int t = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *dx = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x) * RPB + sub; row < a.rows; row += gridDim.x * RPB) {
    const size_t base = static_cast<size_t>(row) * a.R;
    const int head = static_cast<int>(base % VEC);
    const float g = a.gamma ? a.gamma[static_cast<uint32_t>(row) % a.pmod] : 1.f;
    const float mean = a.mean[row];
    const float vpe = a.var[row] + a.eps;
    const float u_dvar = a.dvar ? a.dvar[row] : 0.f;
    const float u_dmean = a.dmean ? a.dmean[row] : 0.f;
    RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      xr[k] = load_piece<T, VEC>(x + base, head, p);
      dr[k] = load_piece<T, VEC>(dy + base, head, p);
    }
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;
    float sdy = 0.f, sdx = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      sdy = raw_sum<T, VEC>(dr[k], sdy);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        sdx = elem_fma<T, VEC>(dr[k], j, xh, sdx);
      }
    }
    row_sum2<TPR>(sdy, sdx, lds);
    if (t == 0) {
      a.ws[2 * static_cast<size_t>(row)] = sdx;
      a.ws[2 * static_cast<size_t>(row) + 1] = sdy;
    }
    if (dx == nullptr) continue;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * (g * sdx) * a.inv_R + (a.dvar ? 2.f * u_dvar * (vpe * istd) * a.inv_R : 0.f);
    const float cb = -(g * sdy) * istd * a.inv_R + (a.dmean ? u_dmean * a.inv_R : 0.f);
    const float gi = g * istd;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          o[j] = elem_fma<T, VEC>(dr[k], j, gi, fmaf(xh, cA, cb));
        }
        store_piece<T, VEC>(dx + base, p, o, a.accum_dx);
      }
    }
  }
}

// GroupNormalization: the channels (within the group) of the first and the last
// element of a piece, and the element of the vector where the second begins
// (VEC when the piece lies inside one channel).
struct PieceChannels {
  uint32_t c0, c1;
  int jb;
};

template <int VEC>
__device__ __forceinline__ PieceChannels piece_channels(const MaskedRowArgs &a, const RowPiece &p) {
  PieceChannels pc;
  const int first = p.col + p.lo, last = p.col + p.hi - 1;
  pc.c0 = p.ok ? a.plane.div(static_cast<uint32_t>(first)) : 0u;
  pc.c1 = p.ok ? a.plane.div(static_cast<uint32_t>(last)) : 0u;
  pc.jb = pc.c1 != pc.c0 ? static_cast<int>((pc.c0 + 1u) * a.plane.d) - p.col : VEC;
  return pc;
}

template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(TPR)
gn_masked_fwd_kernel(const MaskedRowArgs a) {
  static_assert(TPR >= 256, "a block per row");
  __shared__ float lds[2 * 16];
  const int t = threadIdx.x;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x); row < a.rows; row += gridDim.x) {
    const size_t base = static_cast<size_t>(row) * a.R;
    const int head = static_cast<int>(base % VEC);
    const uint32_t pb = (static_cast<uint32_t>(row) % a.pmod) * a.cpg;
    RawVec<T, VEC> raw[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k)
      raw[k] = load_piece<T, VEC>(x + base, head, row_piece<VEC>(a, base, head, k * TPR + t));
    // gamma and beta of the piece's one or two channels, behind the row's loads
    float g0[NL], g1[NL], b0[NL], b1[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const PieceChannels pc = piece_channels<VEC>(a, row_piece<VEC>(a, base, head, k * TPR + t));
      g0[k] = a.gamma ? a.gamma[pb + pc.c0] : 1.f;
      g1[k] = a.gamma ? a.gamma[pb + pc.c1] : 1.f;
      b0[k] = a.beta ? a.beta[pb + pc.c0] : 0.f;
      b1[k] = a.beta ? a.beta[pb + pc.c1] : 0.f;
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
    const float mean = row_sum<TPR>(s, lds) * a.inv_R;
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
          q = (j >= p.lo && j < p.hi) ? fmaf(d, d, q) : q;
        }
      }
    }
    const float var = row_sum<TPR>(q, lds) * a.inv_R;
    const float istd = inv_std(var, a.eps);
    if (t == 0) {
      a.mean[row] = mean;
      a.var[row] = var;
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
        const PieceChannels pc = piece_channels<VEC>(a, p);
        const float gs0 = g0[k] * istd, gs1 = g1[k] * istd;
        const float sh0 = fmaf(-mean, gs0, b0[k]), sh1 = fmaf(-mean, gs1, b1[k]);
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const bool second = j >= pc.jb;
          if constexpr (sizeof(T) == 2) {
            o[j] = elem_fma<T, VEC>(raw[k], j, second ? gs1 : gs0, second ? sh1 : sh0);
          } else {
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), second ? gs1 : gs0, second ? b1[k] : b0[k]);
          }
        }
        store_piece<T, VEC>(y + base, p, o, 0);
      }
    }
  }
}

// GroupNormalization backward.  The 64 vectors a wave holds in one slot meet two
// channels at most (planes of 64 * VEC elements and more): per slot the wave
// adds its lanes' (sum dy*xh, sum dy) for the first of them and for the next,
// a thread per channel then adds the runs that belong to it in slot and wave
// order - the pair per (row, channel) that dgamma / dbeta are summed from - and
// the row's s1 = sum g*sdy, t2 = sum g*sdx follow from those.
template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__(TPR)
gn_masked_bwd_kernel(const MaskedRowArgs a) {
  static_assert(TPR >= 256, "a block per row");
  constexpr int NW = TPR / kWave;
  __shared__ float lds[2 * 16];
  __shared__ float runs[NL * NW * 4]; // per (slot, wave): sdx, sdy of the wave's first channel, of the next
  const int t = threadIdx.x;
  const int wave = t / kWave, lane = t % kWave;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *dx = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x); row < a.rows; row += gridDim.x) {
    const size_t base = static_cast<size_t>(row) * a.R;
    const int head = static_cast<int>(base % VEC);
    const uint32_t pb = (static_cast<uint32_t>(row) % a.pmod) * a.cpg;
    const float mean = a.mean[row];
    const float vpe = a.var[row] + a.eps;
    const float u_dvar = a.dvar ? a.dvar[row] : 0.f;
    const float u_dmean = a.dmean ? a.dmean[row] : 0.f;
    const float g_t = (a.gamma && static_cast<uint32_t>(t) < a.cpg) ? a.gamma[pb + t] : 1.f;
    RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      xr[k] = load_piece<T, VEC>(x + base, head, p);
      dr[k] = load_piece<T, VEC>(dy + base, head, p);
    }
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;
    // the first channel of the wave's run in slot k (the same in every lane)
    auto run_channel = [&](int k) {
      const int first = max((k * TPR + wave * kWave) * VEC - head, 0);
      return a.plane.div(static_cast<uint32_t>(min(first, a.R - 1)));
    };
    lds_barrier(); // runs[] of the previous row has been consumed
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      const PieceChannels pc = piece_channels<VEC>(a, p);
      // the whole piece, then - in the one lane of some hundred whose vector holds
      // a channel boundary - what lies behind the boundary
      float sx0 = 0.f, sy0 = 0.f, sx1 = 0.f, sy1 = 0.f;
      sy0 = raw_sum<T, VEC>(dr[k], 0.f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        sx0 = elem_fma<T, VEC>(dr[k], j, xh, sx0);
      }
      if (pc.jb < VEC) {
#pragma unroll
        for (int j = 1; j < VEC; ++j) {
          if (j >= pc.jb) {
            const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
            const float d = elem_fma<T, VEC>(dr[k], j, a.one, 0.f);
            sx1 = fmaf(d, xh, sx1);
            sy1 += d;
          }
        }
        sx0 -= sx1;
        sy0 -= sy1;
      }
      const uint32_t cw = run_channel(k);
      // the channel of the run's last element: the same for most runs, and then
      // nothing belongs to the next channel
      const int run_last = min((k * TPR + wave * kWave + kWave) * VEC - head, a.R) - 1;
      const bool two = run_last >= 0 && a.plane.div(static_cast<uint32_t>(run_last)) != cw;
      // (a piece outside the row holds zeros: whichever channel takes them)
      const bool first0 = pc.c0 == cw, first1 = pc.c1 == cw;
      float ax = (first0 ? sx0 : 0.f) + ((first1 && pc.jb < VEC) ? sx1 : 0.f);
      float ay = (first0 ? sy0 : 0.f) + ((first1 && pc.jb < VEC) ? sy1 : 0.f);
      float bx = 0.f, by = 0.f;
      ax = wave_sum(ax);
      ay = wave_sum(ay);
      if (two) { // (the same answer in every lane)
        bx = (first0 ? 0.f : sx0) + ((first1 || pc.jb >= VEC) ? 0.f : sx1);
        by = (first0 ? 0.f : sy0) + ((first1 || pc.jb >= VEC) ? 0.f : sy1);
        bx = wave_sum(bx);
        by = wave_sum(by);
      }
      if (lane == 0) {
        float *r = runs + (k * NW + wave) * 4;
        r[0] = ax;
        r[1] = ay;
        r[2] = bx;
        r[3] = by;
      }
    }
    lds_barrier();
    float c1 = 0.f, c2 = 0.f;
    if (static_cast<uint32_t>(t) < a.cpg) {
      // The runs (slot, wave) follow the row's vectors in order: channel t meets
      // the runs of its first to its last vector.
      float sdx = 0.f, sdy = 0.f;
      const int run_lo = (t * static_cast<int>(a.plane.d) + head) / (VEC * kWave);
      const int run_hi = ((t + 1) * static_cast<int>(a.plane.d) - 1 + head) / (VEC * kWave);
      for (int run = run_lo; run <= run_hi; ++run) {
        const int first = max(run * kWave * VEC - head, 0);
        const uint32_t cw = a.plane.div(static_cast<uint32_t>(min(first, a.R - 1)));
        const float *r = runs + run * 4;
        if (cw == static_cast<uint32_t>(t)) {
          sdx += r[0];
          sdy += r[1];
        } else if (cw + 1u == static_cast<uint32_t>(t)) {
          sdx += r[2];
          sdy += r[3];
        }
      }
      const size_t o = 2 * (static_cast<size_t>(row) * a.cpg + t);
      a.ws[o] = sdx;
      a.ws[o + 1] = sdy;
      c1 = g_t * sdy;
      c2 = g_t * sdx;
    }
    row_sum2<TPR>(c1, c2, lds);
    if (dx == nullptr) continue;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * c2 * a.inv_R + (a.dvar ? 2.f * u_dvar * (vpe * istd) * a.inv_R : 0.f);
    const float cb = -c1 * istd * a.inv_R + (a.dmean ? u_dmean * a.inv_R : 0.f);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = row_piece<VEC>(a, base, head, k * TPR + t);
      if (p.ok) {
        const PieceChannels pc = piece_channels<VEC>(a, p);
        const float gi0 = (a.gamma ? a.gamma[pb + pc.c0] : 1.f) * istd;
        const float gi1 = (a.gamma ? a.gamma[pb + pc.c1] : 1.f) * istd;
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          o[j] = elem_fma<T, VEC>(dr[k], j, j >= pc.jb ? gi1 : gi0, fmaf(xh, cA, cb));
        }
        store_piece<T, VEC>(dx + base, p, o, a.accum_dx);
      }
    }
  }
}

// GroupNormalization, a group's planes side by side in one block: TPP threads
// per plane (one wave or more), so a thread's pieces lie inside its plane - no
// channel boundary inside a vector, gamma / beta one scalar per thread - and the
// planes meet only in the sums: per wave through LDS, added in wave order.
// For groups of up to 64 channels whose plane TPP * NL vectors hold
// (channels * TPP threads: a block of 1024 at most).
struct GroupPlanesArgs {
  MaskedRowArgs r;
  int tpp_shift; // threads per plane = 1 << tpp_shift (64 ... 1024)
  int len;       // elements per plane
};

template <int VEC>
__device__ __forceinline__ RowPiece plane_piece(const GroupPlanesArgs &g, size_t base, int head, int v) {
  RowPiece p;
  p.col = v * VEC - head;
  p.ok = p.col < g.len;
  p.lo = p.col < 0 ? -p.col : 0;
  p.hi = min(VEC, g.len - p.col);
  p.tail = static_cast<long long>(base) + p.col + VEC > g.r.total;
  return p;
}

// SUB: 8, 16 or 32 threads per plane (several planes per wave; the sums per
// plane then), 0: whole waves per plane.
template <typename T, int VEC, int NL, int SUB>
__global__ void __launch_bounds__(1024)
gn_planes_masked_fwd_kernel(const GroupPlanesArgs g) {
  const MaskedRowArgs &a = g.r;
  __shared__ float wsum[2][64];
  const int t = threadIdx.x;
  const int wave = t / kWave, lane = t % kWave;
  const int pl = t >> g.tpp_shift, tp = t & ((1 << g.tpp_shift) - 1);
  const int tpp = 1 << g.tpp_shift;
  // the block's partial sums: one per wave, or one per plane
  const int nparts = SUB > 0 ? static_cast<int>(a.cpg) : static_cast<int>(blockDim.x) / kWave;
  const int part = SUB > 0 ? pl : wave;
  const bool writer = SUB > 0 ? tp == 0 : lane == 0;
  auto part_sum = [&](float v) {
    if constexpr (SUB > 0) {
      return group_sum<(SUB > 0 ? SUB : 8)>(v);
    } else {
      return wave_sum(v);
    }
  };
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x); row < a.rows; row += gridDim.x) {
    const size_t base = static_cast<size_t>(row) * a.R + static_cast<size_t>(pl) * g.len;
    const int head = static_cast<int>(base % VEC);
    const uint32_t pc = (static_cast<uint32_t>(row) % a.pmod) * a.cpg + pl;
    const float gam = a.gamma ? a.gamma[pc] : 1.f;
    const float bet = a.beta ? a.beta[pc] : 0.f;
    RawVec<T, VEC> raw[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k)
      raw[k] = load_piece<T, VEC>(x + base, head, plane_piece<VEC>(g, base, head, k * tpp + tp));
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
    s = part_sum(s);
    lds_barrier(); // the previous row's sums have been read
    if (writer) wsum[0][part] = s;
    lds_barrier();
    float tot = 0.f;
    for (int w = 0; w < nparts; ++w) tot += wsum[0][w];
    const float mean = tot * a.inv_R;
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = plane_piece<VEC>(g, base, head, k * tpp + tp);
      if (p.ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
          q = (j >= p.lo && j < p.hi) ? fmaf(d, d, q) : q;
        }
      }
    }
    q = part_sum(q);
    if (writer) wsum[1][part] = q;
    lds_barrier();
    float qt = 0.f;
    for (int w = 0; w < nparts; ++w) qt += wsum[1][w];
    const float var = qt * a.inv_R;
    const float istd = inv_std(var, a.eps);
    if (t == 0) {
      a.mean[row] = mean;
      a.var[row] = var;
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    const float gs = gam * istd;
    const float sh = fmaf(-mean, gs, bet);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = plane_piece<VEC>(g, base, head, k * tpp + tp);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if constexpr (sizeof(T) == 2) {
            o[j] = elem_fma<T, VEC>(raw[k], j, gs, sh);
          } else {
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), gs, bet);
          }
        }
        store_piece<T, VEC>(y + base, p, o, 0);
      }
    }
  }
}

template <typename T, int VEC, int NL, int SUB>
__global__ void __launch_bounds__(1024)
gn_planes_masked_bwd_kernel(const GroupPlanesArgs g) {
  const MaskedRowArgs &a = g.r;
  __shared__ float wsum[64][2]; // per wave (SUB: per plane): sum dy*xh, sum dy
  __shared__ float gch[64];     // gamma of the group's channels
  const int t = threadIdx.x;
  const int wave = t / kWave, lane = t % kWave;
  const int pl = t >> g.tpp_shift, tp = t & ((1 << g.tpp_shift) - 1);
  const int tpp = 1 << g.tpp_shift;
  const int wpp = SUB > 0 ? 1 : tpp / kWave; // partial sums per plane
  const int part = SUB > 0 ? pl : wave;
  const bool writer = SUB > 0 ? tp == 0 : lane == 0;
  auto part_sum = [&](float v) {
    if constexpr (SUB > 0) {
      return group_sum<(SUB > 0 ? SUB : 8)>(v);
    } else {
      return wave_sum(v);
    }
  };
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *dx = static_cast<T *>(a.out);
  for (int row = static_cast<int>(blockIdx.x); row < a.rows; row += gridDim.x) {
    const size_t base = static_cast<size_t>(row) * a.R + static_cast<size_t>(pl) * g.len;
    const int head = static_cast<int>(base % VEC);
    const uint32_t pb = (static_cast<uint32_t>(row) % a.pmod) * a.cpg;
    const float gam = a.gamma ? a.gamma[pb + pl] : 1.f;
    const float g_t = (a.gamma && static_cast<uint32_t>(t) < a.cpg) ? a.gamma[pb + t] : 1.f;
    const float mean = a.mean[row];
    const float vpe = a.var[row] + a.eps;
    const float u_dvar = a.dvar ? a.dvar[row] : 0.f;
    const float u_dmean = a.dmean ? a.dmean[row] : 0.f;
    RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = plane_piece<VEC>(g, base, head, k * tpp + tp);
      xr[k] = load_piece<T, VEC>(x + base, head, p);
      dr[k] = load_piece<T, VEC>(dy + base, head, p);
    }
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;
    float sdy = 0.f, sdx = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      sdy = raw_sum<T, VEC>(dr[k], sdy);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        sdx = elem_fma<T, VEC>(dr[k], j, xh, sdx);
      }
    }
    sdx = part_sum(sdx);
    sdy = part_sum(sdy);
    lds_barrier(); // the previous row's sums have been read
    if (writer) {
      wsum[part][0] = sdx;
      wsum[part][1] = sdy;
    }
    if (static_cast<uint32_t>(t) < a.cpg) gch[t] = g_t;
    lds_barrier();
    // the planes' pairs (the row's share of dgamma / dbeta), a thread per plane
    if (static_cast<uint32_t>(t) < a.cpg) {
      float px = 0.f, py = 0.f;
      for (int w = t * wpp; w < (t + 1) * wpp; ++w) {
        px += wsum[w][0];
        py += wsum[w][1];
      }
      const size_t o = 2 * (static_cast<size_t>(row) * a.cpg + t);
      a.ws[o] = px;
      a.ws[o + 1] = py;
    }
    if (dx == nullptr) continue;
    // the group's s1 = sum g*sdy, t2 = sum g*sdx: planes in order, each plane's waves in order
    float s1 = 0.f, t2 = 0.f;
    for (uint32_t c = 0; c < a.cpg; ++c) {
      float px = 0.f, py = 0.f;
      for (int w = static_cast<int>(c) * wpp; w < static_cast<int>(c + 1) * wpp; ++w) {
        px += wsum[w][0];
        py += wsum[w][1];
      }
      s1 = fmaf(gch[c], py, s1);
      t2 = fmaf(gch[c], px, t2);
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * t2 * a.inv_R + (a.dvar ? 2.f * u_dvar * (vpe * istd) * a.inv_R : 0.f);
    const float cb = -s1 * istd * a.inv_R + (a.dmean ? u_dmean * a.inv_R : 0.f);
    const float gi = gam * istd;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const RowPiece p = plane_piece<VEC>(g, base, head, k * tpp + tp);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          o[j] = elem_fma<T, VEC>(dr[k], j, gi, fmaf(xh, cA, cb));
        }
        store_piece<T, VEC>(dx + base, p, o, a.accum_dx);
      }
    }
  }
}

// BatchNormalization (planes layout) over planes that are no whole number of
// vectors (17 x 17, 35 x 35): a block holds its channel - the N planes (n, c),
// each taken through the tensor's aligned vectors with masked edges as above -
// in registers between the statistics and the normalization: 2 S forward and
// 3 S backward in one launch each, the channel's dgamma / dbeta written by the
// block itself.  The split reduction these shapes took otherwise reads x twice
// through three launches per direction.
struct BnMaskedArgs {
  const void *x;
  const void *dy;
  void *out;
  const float *gamma, *beta;
  float *bmean, *bvar;       // forward: the batch statistics, written
  float *rmean, *rvar;       // forward: running statistics, may be null
  const float *mean, *var;   // backward: read
  const float *dmean, *dvar; // may be null
  float *dgamma, *dbeta;     // may be null
  uint32_t N, C, HW;
  uint32_t nvp; // vectors a plane can meet = (HW + 2 * VEC - 2) / VEC
  FastDiv nvpd;
  long long total;
  float inv_cnt, unbias, decay, eps, one;
  int accum_dx, accum_g, accum_b;
};

// Piece i of channel c: vector i % nvp of plane i / nvp.
template <int VEC>
__device__ __forceinline__ RowPiece bn_piece(const BnMaskedArgs &a, uint32_t c, uint32_t i, size_t &base,
                                             int &head) {
  const uint32_t n = a.nvpd.div(i);
  const uint32_t v = i - n * a.nvp;
  const bool plane = n < a.N;
  base = (static_cast<size_t>(plane ? n : 0u) * a.C + c) * a.HW;
  head = static_cast<int>(base % VEC);
  RowPiece p;
  p.col = static_cast<int>(v) * VEC - head;
  p.ok = plane && p.col < static_cast<int>(a.HW);
  p.lo = p.col < 0 ? -p.col : 0;
  p.hi = min(VEC, static_cast<int>(a.HW) - p.col);
  p.tail = static_cast<long long>(base) + p.col + VEC > a.total;
  return p;
}

// TB threads per block: 1024, or 256 for channels of few vectors (several
// blocks to a CU then, one's sums under another's loads).
template <typename T, int VEC, int NL, int TB>
__global__ void __launch_bounds__(TB)
bn_masked_fwd_kernel(const BnMaskedArgs a) {
  __shared__ float red[TB / kWave];
  const uint32_t t = threadIdx.x;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);
  for (uint32_t c = blockIdx.x; c < a.C; c += gridDim.x) {
    const float gam = a.gamma ? a.gamma[c] : 1.f;
    const float bet = a.beta ? a.beta[c] : 0.f;
    const float rm = a.rmean ? a.rmean[c] : 0.f;
    const float rv = a.rvar ? a.rvar[c] : 0.f;
    RawVec<T, VEC> raw[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      size_t base;
      int head;
      const RowPiece p = bn_piece<VEC>(a, c, k * TB + t, base, head);
      raw[k] = load_piece<T, VEC>(x + base, head, p);
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) s = raw_sum<T, VEC>(raw[k], s);
    const float mean = onchip_block_sum<TB>(s, red) * a.inv_cnt;
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      size_t base;
      int head;
      const RowPiece p = bn_piece<VEC>(a, c, k * TB + t, base, head);
      if (p.ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
          q = (j >= p.lo && j < p.hi) ? fmaf(d, d, q) : q;
        }
      }
    }
    const float var = onchip_block_sum<TB>(q, red) * a.inv_cnt;
    const float istd = inv_std(var, a.eps);
    if (t == 0) {
      a.bmean[c] = mean;
      a.bvar[c] = var;
      if (a.rmean) a.rmean[c] = a.decay * rm + (1.f - a.decay) * mean;
      if (a.rvar) a.rvar[c] = a.decay * rv + (1.f - a.decay) * var * a.unbias;
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);
    const float gs = gam * istd;
    const float sh = fmaf(-mean, gs, bet);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      size_t base;
      int head;
      const RowPiece p = bn_piece<VEC>(a, c, k * TB + t, base, head);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if constexpr (sizeof(T) == 2) {
            o[j] = elem_fma<T, VEC>(raw[k], j, gs, sh);
          } else {
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), gs, bet);
          }
        }
        store_piece<T, VEC>(y + base, p, o, 0);
      }
    }
  }
}

template <typename T, int VEC, int NL, int TB>
__global__ void __launch_bounds__(TB)
bn_masked_bwd_kernel(const BnMaskedArgs a) {
  __shared__ float red[TB / kWave];
  const uint32_t t = threadIdx.x;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *dx = static_cast<T *>(a.out);
  for (uint32_t c = blockIdx.x; c < a.C; c += gridDim.x) {
    const float gam = a.gamma ? a.gamma[c] : 1.f;
    const float mean = a.mean[c];
    const float vpe = a.var[c] + a.eps;
    const float u_dvar = a.dvar ? a.dvar[c] : 0.f;
    const float u_dmean = a.dmean ? a.dmean[c] : 0.f;
    const float old_g = (a.dgamma && a.accum_g) ? a.dgamma[c] : 0.f;
    const float old_b = (a.dbeta && a.accum_b) ? a.dbeta[c] : 0.f;
    RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      size_t base;
      int head;
      const RowPiece p = bn_piece<VEC>(a, c, k * TB + t, base, head);
      xr[k] = load_piece<T, VEC>(x + base, head, p);
      dr[k] = load_piece<T, VEC>(dy + base, head, p);
    }
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;
    float sdy = 0.f, sdx = 0.f;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      sdy = raw_sum<T, VEC>(dr[k], sdy);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        sdx = elem_fma<T, VEC>(dr[k], j, xh, sdx);
      }
    }
    sdx = onchip_block_sum<TB>(sdx, red);
    sdy = onchip_block_sum<TB>(sdy, red);
    if (t == 0) {
      if (a.dgamma) a.dgamma[c] = sdx + old_g;
      if (a.dbeta) a.dbeta[c] = sdy + old_b;
    }
    if (dx == nullptr) continue;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * gam * sdx * a.inv_cnt + (a.dvar ? 2.f * u_dvar * (vpe * istd) * a.inv_cnt : 0.f);
    const float cb = -gam * sdy * istd * a.inv_cnt + (a.dmean ? u_dmean * a.inv_cnt : 0.f);
    const float gi = gam * istd;
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      size_t base;
      int head;
      const RowPiece p = bn_piece<VEC>(a, c, k * TB + t, base, head);
      if (p.ok) {
        float o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          o[j] = elem_fma<T, VEC>(dr[k], j, gi, fmaf(xh, cA, cb));
        }
        store_piece<T, VEC>(dx + base, p, o, a.accum_dx);
      }
    }
  }
}

namespace {

MaskedRowArgs masked_args(const RowProblem &p) {
  MaskedRowArgs a{};
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.ws = static_cast<float *>(p.ws);
  a.rows = static_cast<int>(p.rows);
  a.R = static_cast<int>(p.R);
  a.total = static_cast<long long>(p.rows) * p.R;
  a.pmod = static_cast<uint32_t>(p.bc_gamma ? p.channels : p.rows);
  a.pmod_b = static_cast<uint32_t>(p.bc_beta ? p.channels : p.rows);
  a.plane = FastDiv(static_cast<uint32_t>(p.R));
  a.cpg = 1;
  if (p.mode == kRowGN) {
    a.pmod = a.pmod_b = static_cast<uint32_t>(p.groups);
    a.cpg = static_cast<uint32_t>(p.channels / p.groups);
    a.plane = FastDiv(static_cast<uint32_t>(p.spatial));
  }
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / static_cast<double>(p.R));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  return a;
}

// Threads per row and vectors per thread for rows of up to nv vectors (the
// row's own and the two it shares); ok = false beyond 1024 x 8.
struct MaskedCfg {
  bool ok = false;
  int tpr = 64, nl = 1;
};

// The layout with the fewest idle slots (a slot beyond the row still issues
// its load); among equals the fewest threads.
MaskedCfg pick_masked(int64_t nv, int min_tpr = 8) {
  MaskedCfg c;
  int64_t best = 0;
  // (planes of a few vectors: several rows per wave, at most 4 vectors a thread)
  for (int tpr : {8, 16, 32}) {
    if (tpr < min_tpr) continue;
    for (int nl : {1, 2, 4}) {
      const int64_t cap = static_cast<int64_t>(tpr) * nl;
      if (cap >= nv && (!c.ok || cap < best)) {
        c.ok = true;
        c.tpr = tpr;
        c.nl = nl;
        best = cap;
      }
    }
  }
  if (c.ok) return c;
  for (int tpr : {64, 256, 512, 1024}) {
    if (tpr < min_tpr) continue;
    for (int nl : {1, 2, 3, 4, 5, 6, 8}) {
      const int64_t cap = static_cast<int64_t>(tpr) * nl;
      if (cap >= nv && (!c.ok || cap < best)) {
        c.ok = true;
        c.tpr = tpr;
        c.nl = nl;
        best = cap;
      }
    }
  }
  return c;
}

// The planes-side-by-side layout for a group: threads per plane (a power of two
// from 64) and vectors per thread, fewest idle slots; ok = false when the
// group's channels times the threads of a plane exceed a block.
struct PlanesCfg {
  bool ok = false;
  int tpp_shift = 6, nl = 1; // (shift 3 - 5: several planes per wave)
};

PlanesCfg pick_planes(const RowProblem &p, int vec, bool backward) {
  PlanesCfg c;
  const int64_t cpg = p.channels / p.groups;
  if (cpg > 64 || !tune_int("ROW_MASKED_PLANES", 1)) return c;
  const int64_t nv = (p.spatial + 2 * vec - 2) / vec;
  // The backward holds x and dy: 8 vectors of each are past 128 registers (52 -
  // 64 bytes of spills).  Taken for half data where nothing smaller fits
  // ([8,128,127,127] G=32: 27.6 against 32.1 us through the boundary-splitting
  // kernel; float [16,256,63,63]: 55.8 against 51.8 us, so not there).
  for (int most : {6, 8}) {
    if (most == 8 && backward && p.dtype != NBLAHIP_F16) break;
    int64_t best = 0;
    for (int sh = 3; sh <= 10; ++sh) {
      if ((cpg << sh) > 1024) break;
      for (int nl : {1, 2, 3, 4, 5, 6, 8}) {
        if (sh < 6 && nl != 1 && nl != 2 && nl != 4) continue; // (the sub-wave layouts' cases)
        if (backward && nl > most) continue;
        const int64_t cap = static_cast<int64_t>(nl) << sh;
        if (cap >= nv && (!c.ok || cap < best)) {
          c.ok = true;
          c.tpp_shift = sh;
          c.nl = nl;
          best = cap;
        }
      }
    }
    if (c.ok || !backward) break;
  }
  return c;
}

bool masked_plan(const RowProblem &p, bool backward, MaskedCfg &cfg) {
  if ((p.mode != kRowIN && p.mode != kRowGN) || !tune_int("ROW_MASKED", 1)) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.R < 2 * vec) return false;
  if (!aligned16(p.x) || (p.out && !aligned16(p.out)) || (backward && !aligned16(p.dy))) return false;
  if (p.rows >= (int64_t{1} << 31) / std::max<int64_t>(1, p.R)) return false;
  // Half planes of up to 1024 elements that are a whole number of 8-byte
  // vectors (6 x 6, 10 x 10, 14 x 14 ... 30 x 30): the plain row kernels with
  // those vectors win over the masked 16-byte pieces - InstanceNormalization in
  // both directions (forward + backward us, masked -> plain: [128,512,14,14]
  // 42.3 -> 38.1, [128,2048,6,6] 40.6 -> 31.7, [64,256,26,26] 31.1 -> 26.3,
  // [16,256,30,30] 17.7 -> 12.5), GroupNormalization in the forward
  // ([128,512,14,14] 18.2 -> 13.2, [128,2048,6,6] 25.3 -> 11.6, [16,256,30,30]
  // 8.6 -> 7.1) and, from 129 elements on, in the backward ([128,512,14,14] 32.0
  // -> 21.9, [64,256,26,26] 22.5 -> 20.8; but [128,2048,6,6] 37.4 -> 49.9).
  // Larger planes stay here: [16,256,46,46] InstanceNormalization 23.2 against
  // 38.8 through the row kernels (a block per channel walks the batch), the
  // forwards 3-13 % ahead as well.
  if (p.dtype == NBLAHIP_F16 && p.spatial % 4 == 0 && p.spatial <= 1024 && p.R / 4 <= 8192 &&
      !tune_int("ROW_MASKED_MID", 0)) {
    if (p.mode == kRowIN || !backward || p.spatial > 128) return false;
  }
  if (p.mode == kRowIN) {
    if (p.R % vec == 0) return false; // whole vectors: the plain kernels
    cfg = pick_masked((p.R + 2 * vec - 2) / vec);
    return cfg.ok;
  }
  // groups: planes that are no whole number of vectors, long enough for one
  // channel boundary per vector (backward: two channels per wave-wide run), a
  // thread per channel of the group
  if (p.spatial % vec == 0 || !tune_int("ROW_MASKED_GROUPS", 1)) return false;
  if (p.spatial >= 2 * vec && pick_planes(p, vec, backward).ok) return true; // the planes side by side
  if (p.spatial < (backward ? 64 * vec : vec) || p.channels / p.groups > 256) return false;
  cfg = pick_masked((p.R + 2 * vec - 2) / vec, 256);
  return cfg.ok;
}

template <typename T, int VEC, bool BWD>
int run_group_planes(const PlanesCfg &c, const GroupPlanesArgs &g, int grid, int block, hipStream_t st) {
  const int sub = c.tpp_shift < 6 ? 1 << c.tpp_shift : 0;
#define PLANES_CASE(NL, SUB)                                                                       \
  if (c.nl == (NL) && sub == (SUB)) {                                                              \
    if constexpr (BWD) {                                                                           \
      NBLAHIP_LAUNCH("gn_planes_masked_bwd_kernel", (gn_planes_masked_bwd_kernel<T, VEC, NL, SUB>),\
                     dim3(grid), dim3(block), 0, st, g);                                           \
    } else {                                                                                       \
      NBLAHIP_LAUNCH("gn_planes_masked_fwd_kernel", (gn_planes_masked_fwd_kernel<T, VEC, NL, SUB>),\
                     dim3(grid), dim3(block), 0, st, g);                                           \
    }                                                                                              \
    return last_launch_status();                                                                   \
  }
  PLANES_CASE(1, 0) PLANES_CASE(2, 0) PLANES_CASE(3, 0) PLANES_CASE(4, 0) PLANES_CASE(5, 0)
  PLANES_CASE(6, 0)
  PLANES_CASE(8, 0)
  PLANES_CASE(1, 8) PLANES_CASE(2, 8) PLANES_CASE(4, 8)
  PLANES_CASE(1, 16) PLANES_CASE(2, 16) PLANES_CASE(4, 16)
  PLANES_CASE(1, 32) PLANES_CASE(2, 32) PLANES_CASE(4, 32)
#undef PLANES_CASE
  return NBLAHIP_EINVAL;
}

template <bool BWD>
int launch_group_planes(const RowProblem &p, const PlanesCfg &c, const MaskedRowArgs &a, hipStream_t st) {
  GroupPlanesArgs g{};
  g.r = a;
  g.tpp_shift = c.tpp_shift;
  g.len = static_cast<int>(p.spatial);
  const int block = static_cast<int>((p.channels / p.groups) << c.tpp_shift);
  const int grid = static_cast<int>(std::min<int64_t>(p.rows, 1 << 20));
  return p.dtype == NBLAHIP_F16 ? run_group_planes<__half, 8, BWD>(c, g, grid, block, st)
                                : run_group_planes<float, 4, BWD>(c, g, grid, block, st);
}

template <typename T, int VEC, bool BWD>
int run_masked_groups(const MaskedCfg &c, const MaskedRowArgs &a, int grid, hipStream_t st) {
#define MASKED_CASE(NL, TPR)                                                                       \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                            \
    if constexpr (BWD) {                                                                           \
      NBLAHIP_LAUNCH("gn_masked_bwd_kernel", (gn_masked_bwd_kernel<T, VEC, NL, TPR>), dim3(grid),  \
                     dim3(TPR), 0, st, a);                                                         \
    } else {                                                                                       \
      NBLAHIP_LAUNCH("gn_masked_fwd_kernel", (gn_masked_fwd_kernel<T, VEC, NL, TPR>), dim3(grid),  \
                     dim3(TPR), 0, st, a);                                                         \
    }                                                                                              \
    return last_launch_status();                                                                   \
  }
#define MASKED_TPR(TPR)                                                                 \
  MASKED_CASE(1, TPR) MASKED_CASE(2, TPR) MASKED_CASE(3, TPR) MASKED_CASE(4, TPR)       \
  MASKED_CASE(5, TPR) MASKED_CASE(6, TPR) MASKED_CASE(8, TPR)
  MASKED_TPR(256)
  MASKED_TPR(512)
  MASKED_TPR(1024)
#undef MASKED_TPR
#undef MASKED_CASE
  return NBLAHIP_EINVAL;
}

template <typename T, int VEC, bool BWD>
int run_masked(const MaskedCfg &c, const MaskedRowArgs &a, int grid, hipStream_t st) {
#define MASKED_CASE(NL, TPR)                                                                       \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                            \
    if constexpr (BWD) {                                                                           \
      NBLAHIP_LAUNCH("in_masked_bwd_kernel", (in_masked_bwd_kernel<T, VEC, NL, TPR>), dim3(grid),  \
                     dim3(RowBlock<TPR>::kBlock), 0, st, a);                                       \
    } else {                                                                                       \
      NBLAHIP_LAUNCH("in_masked_fwd_kernel", (in_masked_fwd_kernel<T, VEC, NL, TPR>), dim3(grid),  \
                     dim3(RowBlock<TPR>::kBlock), 0, st, a);                                       \
    }                                                                                              \
    return last_launch_status();                                                                   \
  }
#define MASKED_TPR(TPR)                                                                 \
  MASKED_CASE(1, TPR) MASKED_CASE(2, TPR) MASKED_CASE(3, TPR) MASKED_CASE(4, TPR)       \
  MASKED_CASE(5, TPR) MASKED_CASE(6, TPR) MASKED_CASE(8, TPR)
  MASKED_CASE(1, 8) MASKED_CASE(2, 8) MASKED_CASE(4, 8)
  MASKED_CASE(1, 16) MASKED_CASE(2, 16) MASKED_CASE(4, 16)
  MASKED_CASE(1, 32) MASKED_CASE(2, 32) MASKED_CASE(4, 32)
  MASKED_TPR(64)
  MASKED_TPR(256)
  MASKED_TPR(512)
  MASKED_TPR(1024)
#undef MASKED_TPR
#undef MASKED_CASE
  return NBLAHIP_EINVAL;
}

int masked_grid(int64_t rows, int tpr) {
  const int rpb = tpr < 256 ? 256 / tpr : 1;
  return static_cast<int>(std::min<int64_t>((rows + rpb - 1) / rpb, 1 << 20));
}

} // namespace

bool row_masked_fwd(const RowProblem &p, hipStream_t st, int *status) {
  MaskedCfg c;
  if (!masked_plan(p, false, c)) return false;
  const MaskedRowArgs a = masked_args(p);
  if (p.mode == kRowGN) {
    const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
    if (const PlanesCfg pc = pick_planes(p, vec, false); pc.ok && p.spatial >= 2 * vec) {
      *status = launch_group_planes<false>(p, pc, a, st);
      return true;
    }
    const int grid = static_cast<int>(std::min<int64_t>(p.rows, 1 << 20));
    *status = p.dtype == NBLAHIP_F16 ? run_masked_groups<__half, 8, false>(c, a, grid, st)
                                     : run_masked_groups<float, 4, false>(c, a, grid, st);
    return true;
  }
  const int grid = masked_grid(p.rows, c.tpr);
  *status = p.dtype == NBLAHIP_F16 ? run_masked<__half, 8, false>(c, a, grid, st)
                                   : run_masked<float, 4, false>(c, a, grid, st);
  return true;
}

bool row_masked_bwd(const RowProblem &p, hipStream_t st, int *status) {
  MaskedCfg c;
  if (!masked_plan(p, true, c)) return false;
  const int64_t cpg = p.mode == kRowGN ? p.channels / p.groups : 1;
  if (static_cast<size_t>(p.rows) * cpg * 2 * sizeof(float) > p.ws_bytes) return false;
  const MaskedRowArgs a = masked_args(p);
  if (p.mode == kRowGN) {
    const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
    if (const PlanesCfg pc = pick_planes(p, vec, true); pc.ok && p.spatial >= 2 * vec) {
      *status = launch_group_planes<true>(p, pc, a, st);
      return true;
    }
    const int grid = static_cast<int>(std::min<int64_t>(p.rows, 1 << 20));
    *status = p.dtype == NBLAHIP_F16 ? run_masked_groups<__half, 8, true>(c, a, grid, st)
                                     : run_masked_groups<float, 4, true>(c, a, grid, st);
    return true;
  }
  const int grid = masked_grid(p.rows, c.tpr);
  *status = p.dtype == NBLAHIP_F16 ? run_masked<__half, 8, true>(c, a, grid, st)
                                   : run_masked<float, 4, true>(c, a, grid, st);
  return true;
}

namespace {

// Eligibility and arguments of the masked BatchNormalization kernels; nl =
// vectors per thread, tb = threads per block.
bool bn_masked_args(const BnProblem &p, bool backward, BnMaskedArgs &a, int &nl, int &tb) {
  if (!tune_int("BN_MASKED_ONCHIP", 1)) return false;
  if (p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.size2 % vec == 0 || p.size2 < 2 * vec || p.size0 < 1) return false;
  if (!aligned16(p.x) || (p.out && !aligned16(p.out)) || (backward && !aligned16(p.dy))) return false;
  const int64_t total = p.size0 * p.C * p.size2;
  if (total >= (int64_t{1} << 31)) return false;
  const int64_t nvp = (p.size2 + 2 * vec - 2) / vec;
  const int64_t pieces = p.size0 * nvp;
  // (beyond: x, or x and dy, no longer fit the registers of a 1024-thread block)
  const int most = backward ? 5 : (p.dtype == NBLAHIP_F16 ? 8 : 6);
  tb = (pieces + 255) / 256 <= most ? 256 : kOnchipBlock;
  nl = static_cast<int>((pieces + tb - 1) / tb);
  if (nl > most) return false;
  // (fewer channels than this share of the CUs: most of the chip would idle)
  if (p.C * 100 < static_cast<int64_t>(device_cus()) * tune_int("BN_MASKED_ONCHIP_MIN_PCT", 1)) return false;
  a = BnMaskedArgs{};
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.bmean = p.batch_mean;
  a.bvar = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.dgamma = p.dgamma;
  a.dbeta = p.dbeta;
  a.N = static_cast<uint32_t>(p.size0);
  a.C = static_cast<uint32_t>(p.C);
  a.HW = static_cast<uint32_t>(p.size2);
  a.nvp = static_cast<uint32_t>(nvp);
  a.nvpd = FastDiv(a.nvp);
  a.total = total;
  const double cnt = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  a.inv_cnt = static_cast<float>(1.0 / cnt);
  a.unbias = static_cast<float>(cnt / std::max(cnt - 1.0, 1.0));
  a.decay = p.decay;
  a.eps = p.eps;
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  a.accum_g = p.accum_g;
  a.accum_b = p.accum_b;
  return true;
}

template <typename T, int VEC, bool BWD, int TB>
int run_bn_masked(int nl, const BnMaskedArgs &a, unsigned grid, hipStream_t st) {
#define BN_MASKED_CASE(NL)                                                                         \
  if (nl <= (NL)) {                                                                                \
    if constexpr (BWD) {                                                                           \
      NBLAHIP_LAUNCH("bn_masked_bwd_kernel", (bn_masked_bwd_kernel<T, VEC, NL, TB>), dim3(grid),   \
                     dim3(TB), 0, st, a);                                                          \
    } else {                                                                                       \
      NBLAHIP_LAUNCH("bn_masked_fwd_kernel", (bn_masked_fwd_kernel<T, VEC, NL, TB>), dim3(grid),   \
                     dim3(TB), 0, st, a);                                                          \
    }                                                                                              \
    return last_launch_status();                                                                   \
  }
  BN_MASKED_CASE(1) BN_MASKED_CASE(2) BN_MASKED_CASE(3) BN_MASKED_CASE(4) BN_MASKED_CASE(5)
  if constexpr (!BWD) {
    BN_MASKED_CASE(6)
    if constexpr (sizeof(T) == 2) {
      BN_MASKED_CASE(8)
    }
  }
#undef BN_MASKED_CASE
  return NBLAHIP_EINVAL;
}

template <bool BWD>
int launch_bn_masked(const BnProblem &p, int nl, int tb, const BnMaskedArgs &a, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>(p.C, 1 << 20));
  if (p.dtype == NBLAHIP_F16)
    return tb == 256 ? run_bn_masked<__half, 8, BWD, 256>(nl, a, grid, st)
                     : run_bn_masked<__half, 8, BWD, kOnchipBlock>(nl, a, grid, st);
  return tb == 256 ? run_bn_masked<float, 4, BWD, 256>(nl, a, grid, st)
                   : run_bn_masked<float, 4, BWD, kOnchipBlock>(nl, a, grid, st);
}

} // namespace

bool bn_masked_takes(const BnProblem &p, bool backward) {
  BnMaskedArgs a;
  int nl = 0, tb = 0;
  return bn_masked_args(p, backward, a, nl, tb);
}

bool bn_masked_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  BnMaskedArgs a;
  int nl = 0, tb = 0;
  if (!p.out || !p.batch_mean || !p.batch_var || !bn_masked_args(p, false, a, nl, tb)) return false;
  *status = launch_bn_masked<false>(p, nl, tb, a, st);
  return true;
}

bool bn_masked_bwd(const BnProblem &p, hipStream_t st, int *status) {
  BnMaskedArgs a;
  int nl = 0, tb = 0;
  if (!p.batch_stat || !p.mean || !p.var || !bn_masked_args(p, true, a, nl, tb)) return false;
  *status = launch_bn_masked<true>(p, nl, tb, a, st);
  return true;
}

} // namespace nblahip
