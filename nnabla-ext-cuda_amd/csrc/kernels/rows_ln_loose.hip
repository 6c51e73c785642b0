// LayerNormalization backward over rows that are no whole number of 16-byte
// vectors, or that do not start on a 16-byte boundary (a hidden size of 1023,
// 1000 or 1028 half elements; a tensor view at an odd offset).  The row kernels
// of rows.cuh take such rows with scalar loads - eight times the memory
// instructions for half data, none of the packed arithmetic: 3.8 copies' time
// for the backward of [16384, 1023] half where 1024 takes 1.7.
//
// Here a thread keeps the columns it has in rows.cuh - vector k*64 + lane of
// every row, so its per-column gamma and gradient accumulators stay put from
// row to row - and reads them with 16-byte accesses at element alignment, which
// the memory pipeline of this GPU takes for global memory (a plain copy loses
// 7 % to it; in this kernel, whose waves wait for every row, the extra line per
// wave-wide access costs more: 24.4 us for [16384, 1023] half against 18.9 for
// 1024).  The elements a row has beyond its last whole vector (fewer than VEC)
// are one lane's: read as the tail of the vector that ends where the row ends,
// written element by element, so nothing is touched outside the tensor.
//
// Only the backward, and only the wave-per-row layouts (rows of up to 256
// vectors), are kept: measured on [16384, 1023] / [16384, 1028] half and
// [16384, 1023] float the backward takes 31 / 42 / 47 us against 54 / 54 / 60
// through the scalar rows, but the forward (whose waves do one row each, so that
// the parameter loads ahead of the row are paid per row) came out at 27 - 30 us
// against 24 / 20 / 29, and block-per-row layouts lost in both directions
// ([8192, 4100] half 87 against 83 us).
#include <algorithm>

#include "rows_dispatch.hpp"

namespace nblahip {

namespace {

// A 16-byte vector at element alignment: the load and the store carry the
// element's alignment, so the compiler assumes no more than that of the address.
typedef uint32_t loose_u4 __attribute__((ext_vector_type(4), aligned(2)));
typedef float loose_f4 __attribute__((ext_vector_type(4), aligned(4)));

template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> load_loose(const T *__restrict__ p) {
  RawVec<T, VEC> r;
  if constexpr (sizeof(T) == 4) {
    static_assert(VEC == 4, "16-byte vectors");
    const loose_f4 v = *reinterpret_cast<const loose_f4 *>(p);
    r.v = make_float4(v.x, v.y, v.z, v.w);
  } else {
    static_assert(VEC == 8, "16-byte vectors");
    const loose_u4 v = *reinterpret_cast<const loose_u4 *>(p);
    r.v = make_uint4(v.x, v.y, v.z, v.w);
  }
  return r;
}

template <typename T, int VEC>
__device__ __forceinline__ void store_loose(T *__restrict__ p, const float (&o)[VEC]) {
  if constexpr (sizeof(T) == 4) {
    const loose_f4 v = {o[0], o[1], o[2], o[3]};
    __builtin_nontemporal_store(v, reinterpret_cast<loose_f4 *>(p));
  } else {
    uint4 raw;
    __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) h[i] = __floats2half2_rn(o[2 * i], o[2 * i + 1]);
    const loose_u4 v = {raw.x, raw.y, raw.z, raw.w};
    __builtin_nontemporal_store(v, reinterpret_cast<loose_u4 *>(p));
  }
}

// Elements e .. VEC-1 of v moved down to 0 .. VEC-1-e, zeros behind them
// (0 <= e < VEC, the same for every lane: the branches are scalar).
template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> shift_down(RawVec<T, VEC> v, int e) {
  if constexpr (sizeof(T) == 4) {
    float4 o = v.v;
    if (e == 0) {
    } else if (e == 1) {
      o = make_float4(v.v.y, v.v.z, v.v.w, 0.f);
    } else if (e == 2) {
      o = make_float4(v.v.z, v.v.w, 0.f, 0.f);
    } else {
      o = make_float4(v.v.w, 0.f, 0.f, 0.f);
    }
    v.v = o;
  } else {
    unsigned long long lo = (static_cast<unsigned long long>(v.v.y) << 32) | v.v.x;
    unsigned long long hi = (static_cast<unsigned long long>(v.v.w) << 32) | v.v.z;
    const int bits = 16 * e;
    if (bits == 0) {
    } else if (bits >= 64) {
      lo = bits == 64 ? hi : hi >> (bits - 64);
      hi = 0;
    } else {
      lo = (lo >> bits) | (hi << (64 - bits));
      hi >>= bits;
    }
    v.v = make_uint4(static_cast<uint32_t>(lo), static_cast<uint32_t>(lo >> 32),
                     static_cast<uint32_t>(hi), static_cast<uint32_t>(hi >> 32));
  }
  return v;
}

template <typename T, int VEC>
__device__ __forceinline__ RawVec<T, VEC> raw_select(bool take, const RawVec<T, VEC> &a,
                                                     const RawVec<T, VEC> &b) {
  RawVec<T, VEC> r;
  if constexpr (sizeof(T) == 4) {
    r.v = make_float4(take ? a.v.x : b.v.x, take ? a.v.y : b.v.y, take ? a.v.z : b.v.z,
                      take ? a.v.w : b.v.w);
  } else {
    r.v = make_uint4(take ? a.v.x : b.v.x, take ? a.v.y : b.v.y, take ? a.v.z : b.v.z,
                     take ? a.v.w : b.v.w);
  }
  return r;
}

template <typename T, int VEC>
__device__ __forceinline__ void store_head(T *__restrict__ p, const float (&o)[VEC], int n) {
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    if (j < n) p[j] = from_f32<T>(o[j]);
}

// Per-column parameters of slot `vi` (n of its VEC columns exist; `fill` for
// the others), with no load behind a per-lane branch - such a load is waited
// for inside its branch, and four of them ahead of the row cost four memory
// round trips.  Whole slots read vectors at a slot index clamped to the row;
// the slot that holds the row's end (`last`: the same for all lanes of the
// block) reads element by element at indices clamped to the row.
template <int VEC>
__device__ __forceinline__ void load_cols(const float *__restrict__ p, int vi, int n, bool last,
                                          int R, float fill, float (&out)[VEC]) {
  if (p == nullptr) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[j] = fill;
  } else if (!last) {
    float v[VEC];
    load_param_vec<VEC>(p + min(vi, R / VEC - 1) * VEC, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[j] = n == VEC ? v[j] : fill;
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float v = p[min(vi * VEC + j, R - 1)];
      out[j] = j < n ? v : fill;
    }
  }
}

// Backward.  Layout and partials as row_bwd_kernel<T, VEC, NL, TPR, kRowLN>:
// a persistent grid, per-column accumulators in registers, the row groups of a
// block folded through LDS, ws[block][0][R] = sum_rows dy*xh and
// ws[block][1][R] = sum_rows dy for ln_param_reduce_kernel.  The padding of the
// last vector holds dy = 0, which keeps it out of every sum.
template <typename T, int VEC, int NL, int TPR>
__global__ void __launch_bounds__((RowBwdBlock<TPR, kRowLN>::kBlock))
ln_loose_bwd_kernel(const RowArgs a) {
  constexpr int RPB = RowBwdBlock<TPR, kRowLN>::kRowsPerBlock;
  constexpr bool KEEP = NL * VEC <= 16;
  __shared__ float lds[2 * 16];
  __shared__ float xfold[RPB > 1 ? 2 * NL * (RPB / 2) * TPR * VEC : 1];
  const int t = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.out);
  const int nfull = a.R / VEC;
  const int tail = a.R - nfull * VEC;
  const int kt = nfull / TPR;
  const bool mine = tail > 0 && t == nfull - kt * TPR;

  float acc_g[NL][VEC], acc_b[NL][VEC], gcol[NL][VEC];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc_g[k][j] = acc_b[k][j] = 0.f;
    const int vi = k * TPR + t;
    load_cols<VEC>(a.gamma, vi, vi < nfull ? VEC : (vi == nfull ? tail : 0), tail > 0 && k == kt,
                   a.R, 1.f, gcol[k]);
  }

  for (int row = static_cast<int>(blockIdx.x) * RPB + sub; row < a.rows;
       row += static_cast<int>(gridDim.x) * RPB) {
    const size_t base = static_cast<size_t>(row) * a.R;
    // (the vectors that end where the row ends, asked for first)
    const RawVec<T, VEC> lastx = load_loose<T, VEC>(x + base + a.R - VEC);
    const RawVec<T, VEC> lastd = load_loose<T, VEC>(dy + base + a.R - VEC);
    RawVec<T, VEC> xr[NL], dr[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int vi = k * TPR + t;
      const bool ok = vi < nfull;
      const size_t at = base + (ok ? vi * VEC : 0);
      xr[k] = raw_or_zero<T, VEC>(ok, load_loose<T, VEC>(x + at));
      dr[k] = raw_or_zero<T, VEC>(ok, load_loose<T, VEC>(dy + at));
    }
    {
      const RawVec<T, VEC> ex = shift_down<T, VEC>(lastx, tail > 0 ? VEC - tail : 0);
      const RawVec<T, VEC> ed = shift_down<T, VEC>(lastd, tail > 0 ? VEC - tail : 0);
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        xr[k] = raw_select<T, VEC>(mine && k == kt, ex, xr[k]);
        dr[k] = raw_select<T, VEC>(mine && k == kt, ed, dr[k]);
      }
    }
    const float mean = a.mean[row];
    const float vpe = a.var[row] + a.eps;
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;

    float s1 = 0.f, t2 = 0.f;
    float xh_keep[KEEP ? NL : 1][VEC], dg_keep[KEEP ? NL : 1][VEC];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
        const float dg = elem_fma<T, VEC>(dr[k], j, gcol[k][j], 0.f);
        acc_g[k][j] = elem_fma<T, VEC>(dr[k], j, xh, acc_g[k][j]);
        acc_b[k][j] = elem_fma<T, VEC>(dr[k], j, a.one, acc_b[k][j]);
        s1 += dg;
        t2 = fmaf(dg, xh, t2);
        if constexpr (KEEP) {
          xh_keep[k][j] = xh;
          dg_keep[k][j] = dg;
        }
      }
    }
    row_sum2<TPR>(s1, t2, lds);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * t2 * a.inv_R +
                     (a.dvar ? 2.f * a.dvar[row] * (vpe * istd) * a.inv_R : 0.f);
    const float cb = -s1 * istd * a.inv_R + (a.dmean ? a.dmean[row] * a.inv_R : 0.f);

    if (dx != nullptr) {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const int vi = k * TPR + t;
        const int n = vi < nfull ? VEC : (vi == nfull ? tail : 0);
        if (n > 0) {
          float o[VEC];
          if constexpr (KEEP) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              o[j] = fmaf(dg_keep[k][j], istd, fmaf(xh_keep[k][j], cA, cb));
          } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
              o[j] = elem_fma<T, VEC>(dr[k], j, gcol[k][j] * istd, fmaf(xh, cA, cb));
            }
          }
          T *dst = dx + base + vi * VEC;
          if (a.accum_dx) {
            // (the row's end: the vector that ends there, shifted - no load
            // behind a per-lane branch; the other lanes read their own vector)
            const bool end = n < VEC;
            RawVec<T, VEC> prev = load_loose<T, VEC>(end ? dx + base + a.R - VEC : dst);
            if (tail > 0 && k == kt) prev = raw_select<T, VEC>(end, shift_down<T, VEC>(prev, VEC - tail), prev);
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = elem_fma<T, VEC>(prev, j, a.one, o[j]);
          }
          if (n == VEC) {
            store_loose<T, VEC>(dst, o);
          } else {
            store_head<T, VEC>(dst, o, n);
          }
        }
      }
    }
  }

  // Fold the RPB row groups of the block into group 0 (a halving tree, fixed
  // order), then write the block's partial [2][R].
  float *wsb = a.ws + static_cast<size_t>(blockIdx.x) * 2 * a.R;
  if constexpr (RPB > 1) {
    constexpr int kSlab = (RPB / 2) * TPR * VEC;
#pragma unroll
    for (int half = RPB / 2; half >= 1; half /= 2) {
      lds_barrier();
      if (sub >= half && sub < 2 * half) {
#pragma unroll
        for (int k = 0; k < NL; ++k) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            xfold[(2 * k) * kSlab + ((sub - half) * TPR + t) * VEC + j] = acc_g[k][j];
            xfold[(2 * k + 1) * kSlab + ((sub - half) * TPR + t) * VEC + j] = acc_b[k][j];
          }
        }
      }
      lds_barrier();
      if (sub < half) {
#pragma unroll
        for (int k = 0; k < NL; ++k) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            acc_g[k][j] += xfold[(2 * k) * kSlab + (sub * TPR + t) * VEC + j];
            acc_b[k][j] += xfold[(2 * k + 1) * kSlab + (sub * TPR + t) * VEC + j];
          }
        }
      }
    }
  }
  if (sub == 0) {
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int vi = k * TPR + t;
      const int n = vi < nfull ? VEC : (vi == nfull ? tail : 0);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if (j < n) {
          wsb[vi * VEC + j] = acc_g[k][j];
          wsb[static_cast<size_t>(a.R) + vi * VEC + j] = acc_b[k][j];
        }
      }
    }
  }
}

#define LOOSE_BWD_CASE(T, NL, TPR)                                                              \
  if (cfg.nl == (NL) && cfg.tpr == (TPR)) {                                                     \
    NBLAHIP_LAUNCH("ln_loose_bwd_kernel", (ln_loose_bwd_kernel<T, FullVec<T>::value, NL, TPR>), \
                   dim3(grid), dim3(RowBwdBlock<TPR, kRowLN>::kBlock), 0, st, a);               \
    return last_launch_status();                                                                \
  }

template <typename T> int run_bwd(const RowCfg &cfg, const RowArgs &a, int grid, hipStream_t st) {
  LOOSE_BWD_CASE(T, 1, 64) LOOSE_BWD_CASE(T, 2, 64) LOOSE_BWD_CASE(T, 4, 64)
  return NBLAHIP_EINVAL;
}

} // namespace

// Takes the backward of LayerNormalization rows of 64 to 256 vectors that the
// aligned 16-byte layouts do not (vec: what row_vec found); gamma must be
// 16-byte aligned itself (it is an array of its own).
bool ln_loose_bwd_wanted(const RowProblem &p, int vec) {
  if (p.mode != kRowLN || !tune_int("LN_LOOSE", 1)) return false;
  const int full = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (vec == full) return false;
  if (p.R < 64 * full || p.R > 256 * full) return false;
  const size_t esize = p.dtype == NBLAHIP_F16 ? 2 : 4;
  auto elem_aligned = [&](const void *q) { return reinterpret_cast<uintptr_t>(q) % esize == 0; };
  if (!elem_aligned(p.x) || (p.out && !elem_aligned(p.out)) || !elem_aligned(p.dy)) return false;
  if (p.gamma && !aligned16(p.gamma)) return false;
  return true;
}

int ln_loose_bwd(const RowProblem &p, const RowArgs &a, const RowCfg &cfg, int grid, hipStream_t st) {
  return p.dtype == NBLAHIP_F16 ? run_bwd<__half>(cfg, a, grid, st) : run_bwd<float>(cfg, a, grid, st);
}

} // namespace nblahip
