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
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
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
MaskedCfg pick_masked(int64_t nv) {
  MaskedCfg c;
  int64_t best = 0;
  for (int tpr : {64, 256, 512, 1024}) {
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

bool masked_plan(const RowProblem &p, bool backward, MaskedCfg &cfg) {
  if (p.mode != kRowIN || !tune_int("ROW_MASKED", 1)) return false;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.R % vec == 0 || p.R < 2 * vec) return false; // whole vectors: the plain kernels
  if (!aligned16(p.x) || (p.out && !aligned16(p.out)) || (backward && !aligned16(p.dy))) return false;
  if (p.rows >= (int64_t{1} << 31) / std::max<int64_t>(1, p.R)) return false;
  cfg = pick_masked((p.R + 2 * vec - 2) / vec);
  return cfg.ok;
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
  const int grid = masked_grid(p.rows, c.tpr);
  *status = p.dtype == NBLAHIP_F16 ? run_masked<__half, 8, false>(c, a, grid, st)
                                   : run_masked<float, 4, false>(c, a, grid, st);
  return true;
}

bool row_masked_bwd(const RowProblem &p, hipStream_t st, int *status) {
  MaskedCfg c;
  if (!masked_plan(p, true, c)) return false;
  if (static_cast<size_t>(p.rows) * 2 * sizeof(float) > p.ws_bytes) return false;
  const MaskedRowArgs a = masked_args(p);
  const int grid = masked_grid(p.rows, c.tpr);
  *status = p.dtype == NBLAHIP_F16 ? run_masked<__half, 8, true>(c, a, grid, st)
                                   : run_masked<float, 4, true>(c, a, grid, st);
  return true;
}

} // namespace nblahip
