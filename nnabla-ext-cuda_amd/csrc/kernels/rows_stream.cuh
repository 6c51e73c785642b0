// Streaming (any row length, any alignment) versions of the row
// normalizations.  Used when a row does not fit the register-cached kernels
// of rows.cuh or the shape breaks their alignment rules.  x is read once for
// the statistics (single-pass Welford, Chan merges across threads) and once
// more for the apply step; a row that was just reduced by one block is
// normally still in that XCD's L2 for the second read.
#pragma once

#include "common.cuh"
#include "rows.cuh"

namespace nblahip {

constexpr int kStreamBlock = 256;

// mean/var of each row; one block per row (grid-stride over blockIdx.x).
// gridDim.y = S > 1 splits every row into S runs of vectors, for tensors of a
// few very long rows (3-D InstanceNormalization, GroupNormalization with one
// group): block (., s) then leaves its Welford state in part[row][s][3] and
// row_stats_merge_kernel finishes.
template <typename T, int VEC>
__global__ void __launch_bounds__(kStreamBlock)
row_stats_stream_kernel(const T *__restrict__ x, int rows, int R, float inv_R,
                        float *__restrict__ mean, float *__restrict__ var,
                        float *__restrict__ part) {
  __shared__ float lds[3 * (kStreamBlock / kWave)];
  constexpr int U = 4;
  const int nv_row = R / VEC;
  const int S = gridDim.y;
  const int chunk = (nv_row + S - 1) / S;
  const int vbegin = static_cast<int>(blockIdx.y) * chunk;
  const int nv = min(nv_row, vbegin + chunk);
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const T *xr = x + static_cast<size_t>(row) * R;
    Welford w{0.f, 0.f, 0.f};
    for (int v0 = vbegin + threadIdx.x; v0 < nv; v0 += kStreamBlock * U) {
      float vals[U * VEC];
      int cnt = 0;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = v0 + u * kStreamBlock;
        float tmp[VEC];
        if (v < nv) {
          load_vec<T, VEC>(xr + static_cast<size_t>(v) * VEC, tmp);
          cnt += VEC;
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) tmp[j] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) vals[u * VEC + j] = tmp[j];
      }
      welford_add_chunk<U * VEC>(w, vals, cnt);
    }
    w = block_welford(w, lds);
    if (threadIdx.x == 0) {
      if (S == 1) {
        mean[row] = w.mean;
        var[row] = w.m2 * inv_R;
      } else {
        float *o = part + 3 * (static_cast<size_t>(row) * S + blockIdx.y);
        o[0] = w.mean;
        o[1] = w.m2;
        o[2] = w.n;
      }
    }
    lds_barrier();
  }
}

// Chan merge of the S partial states of each row, in split order.
__global__ void __launch_bounds__(64)
row_stats_merge_kernel(const float *__restrict__ part, int rows, int S, float inv_R,
                       float *__restrict__ mean, float *__restrict__ var) {
  const int row = blockIdx.x * 64 + threadIdx.x;
  if (row >= rows) return;
  Welford w{0.f, 0.f, 0.f};
  for (int s = 0; s < S; ++s) {
    const float *q = part + 3 * (static_cast<size_t>(row) * S + s);
    w = welford_merge(w, Welford{q[0], q[1], q[2]});
  }
  mean[row] = w.mean;
  var[row] = w.m2 * inv_R;
}

// y = (x-mean[row])*gamma[p]*istd[row] + beta[p] over the whole tensor.
// nvr = vectors per row.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
row_apply_fwd_kernel(const RowArgs a, FastDiv nvr, uint32_t total_vec) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total_vec; i += gridDim.x * 256u) {
    const uint32_t row = nvr.div(i);
    const uint32_t col = (i - row * nvr.d) * VEC;
    const float mean = a.mean[row];
    const float istd = inv_std(a.var[row], a.eps);
    float v[VEC], o[VEC];
    load_vec<T, VEC>(x + static_cast<size_t>(i) * VEC, v);
    if (a.percol) {
      // gamma/beta of VEC columns in one or two 16-byte loads each (vectors
      // are only used when the parameter pointers are aligned)
      float gv[VEC], bv[VEC];
      if (a.gamma) {
        load_param_vec<VEC>(a.gamma + col, gv);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) gv[j] = 1.f;
      }
      if (a.beta) {
        load_param_vec<VEC>(a.beta + col, bv);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) bv[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = (v[j] - mean) * (gv[j] * istd) + bv[j];
    } else {
      // VEC divides the parameter run length, so one index serves the vector.
      const uint32_t poff = a.pdiv.div(col);
      const float g = (a.gamma ? a.gamma[(row % a.pmod) * a.pmul + poff] : 1.f) * istd;
      const float b = a.beta ? a.beta[(row % a.pmod_b) * a.pmul + poff] : 0.f;
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = (v[j] - mean) * g + b;
    }
    store_vec<T, VEC>(y + static_cast<size_t>(i) * VEC, o);
  }
}

// Per-row (s1, t2) for LayerNormalization: s1 = sum dy*gamma[col],
// t2 = sum dy*gamma[col]*(x-mean).  rs[2*row], rs[2*row+1].
template <typename T, int VEC>
__global__ void __launch_bounds__(kStreamBlock)
ln_row_sums_stream_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                          const float *__restrict__ gamma,
                          const float *__restrict__ mean, int rows, int R,
                          float *__restrict__ rs) {
  __shared__ float lds[2 * (kStreamBlock / kWave)];
  // gridDim.y = S > 1: every row in S runs of vectors, partial pairs to
  // rs[(row*S + s)*2] (a partial buffer then), summed by pair_split_merge_kernel.
  const int nv_row = R / VEC;
  const int S = gridDim.y;
  const int chunk = (nv_row + S - 1) / S;
  const int vbegin = static_cast<int>(blockIdx.y) * chunk;
  const int nv = min(nv_row, vbegin + chunk);
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const size_t base = static_cast<size_t>(row) * R;
    const float m = mean[row];
    float s1 = 0.f, t2 = 0.f;
    for (int v = vbegin + threadIdx.x; v < nv; v += kStreamBlock) {
      float xv[VEC], dv[VEC];
      load_vec<T, VEC>(x + base + static_cast<size_t>(v) * VEC, xv);
      load_vec<T, VEC>(dy + base + static_cast<size_t>(v) * VEC, dv);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float dg = dv[j] * (gamma ? gamma[v * VEC + j] : 1.f);
        s1 += dg;
        t2 += dg * (xv[j] - m);
      }
    }
    block_sum2(s1, t2, lds);
    if (threadIdx.x == 0) {
      const size_t o = 2 * (static_cast<size_t>(row) * S + blockIdx.y);
      rs[o] = s1;
      rs[o + 1] = t2;
    }
    lds_barrier();
  }
}

// Per-plane sums for Instance/GroupNormalization: plane p = (n, c) of length L,
// statistics row = p / sdiv.  pairs[2p] = sum dy*(x-mean), pairs[2p+1] = sum dy.
template <typename T, int VEC>
__global__ void __launch_bounds__(kStreamBlock)
plane_sums_stream_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                         const float *__restrict__ mean, int planes, int L,
                         uint32_t sdiv, float *__restrict__ pairs) {
  __shared__ float lds[2 * (kStreamBlock / kWave)];
  // gridDim.y = S > 1: every plane in S runs of vectors, partial pairs to
  // pairs[(p*S + s)*2] (the caller passes a partial buffer then) and
  // pair_split_merge_kernel adds them up.
  const int nv_plane = L / VEC;
  const int S = gridDim.y;
  const int chunk = (nv_plane + S - 1) / S;
  const int vbegin = static_cast<int>(blockIdx.y) * chunk;
  const int nv = min(nv_plane, vbegin + chunk);
  for (int p = blockIdx.x; p < planes; p += gridDim.x) {
    const size_t base = static_cast<size_t>(p) * L;
    const float m = mean[static_cast<uint32_t>(p) / sdiv];
    float sdx = 0.f, sdy = 0.f;
    for (int v = vbegin + threadIdx.x; v < nv; v += kStreamBlock) {
      float xv[VEC], dv[VEC];
      load_vec<T, VEC>(x + base + static_cast<size_t>(v) * VEC, xv);
      load_vec<T, VEC>(dy + base + static_cast<size_t>(v) * VEC, dv);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        sdy += dv[j];
        sdx += dv[j] * (xv[j] - m);
      }
    }
    block_sum2(sdx, sdy, lds);
    if (threadIdx.x == 0) {
      const size_t o = 2 * (static_cast<size_t>(p) * S + blockIdx.y);
      pairs[o] = sdx;
      pairs[o + 1] = sdy;
    }
    lds_barrier();
  }
}

// Sum of the S partial pairs of each plane, in split order.
__global__ void __launch_bounds__(64)
pair_split_merge_kernel(const float *__restrict__ part, int planes, int S,
                        float *__restrict__ pairs) {
  const int p = blockIdx.x * 64 + threadIdx.x;
  if (p >= planes) return;
  float a = 0.f, b = 0.f;
  for (int s = 0; s < S; ++s) {
    a += part[2 * (static_cast<size_t>(p) * S + s)];
    b += part[2 * (static_cast<size_t>(p) * S + s) + 1];
  }
  pairs[2 * static_cast<size_t>(p)] = a;
  pairs[2 * static_cast<size_t>(p) + 1] = b;
}

// From per-plane sums to per-statistics-row (s1, t2), weighting each plane with
// its gamma; also rescales pairs[2p] by istd so that it is the dgamma part.
//   stat row r owns planes [r*ppr, (r+1)*ppr); gamma index of plane p:
//   gmod == 0 : p (per-sample parameter)   else p % gmod (broadcast over batch)
__global__ void __launch_bounds__(64)
plane_to_row_factors_kernel(float *__restrict__ pairs, const float *__restrict__ gamma,
                            const float *__restrict__ var, int rows, int ppr,
                            uint32_t gmod, float eps, float *__restrict__ rs) {
  for (int r = blockIdx.x; r < rows; r += gridDim.x) {
    const float istd = inv_std(var[r], eps);
    float s1 = 0.f, t2 = 0.f;
    for (int c = threadIdx.x; c < ppr; c += 64) {
      const uint32_t p = static_cast<uint32_t>(r) * ppr + c;
      const float g = gamma ? gamma[gmod ? p % gmod : p] : 1.f;
      const float sdx = pairs[2 * static_cast<size_t>(p)];
      s1 += g * pairs[2 * static_cast<size_t>(p) + 1];
      t2 += g * sdx;
      pairs[2 * static_cast<size_t>(p)] = sdx * istd;
    }
    s1 = wave_sum(s1);
    t2 = wave_sum(t2);
    if (threadIdx.x == 0) {
      rs[2 * static_cast<size_t>(r)] = s1;
      rs[2 * static_cast<size_t>(r) + 1] = t2;
    }
  }
}

// dx = dy*gamma[p]*istd + ca*(x-mean) + cb, elementwise over the tensor.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
row_bwd_dx_kernel(const RowArgs a, const float *__restrict__ rs, FastDiv nvr,
                  uint32_t total_vec) {
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.out);
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total_vec; i += gridDim.x * 256u) {
    const uint32_t row = nvr.div(i);
    const uint32_t col = (i - row * nvr.d) * VEC;
    const float mean = a.mean[row];
    const float istd = inv_std(a.var[row], a.eps);
    const float s1 = rs[2 * static_cast<size_t>(row)];
    const float t2 = rs[2 * static_cast<size_t>(row) + 1];
    const float ca = -t2 * istd * istd * istd * a.inv_R +
                     (a.dvar ? 2.f * a.dvar[row] * a.inv_R : 0.f);
    const float cb = -s1 * istd * a.inv_R + (a.dmean ? a.dmean[row] * a.inv_R : 0.f);
    float xv[VEC], dv[VEC], o[VEC];
    load_vec<T, VEC>(x + static_cast<size_t>(i) * VEC, xv);
    load_vec<T, VEC>(dy + static_cast<size_t>(i) * VEC, dv);
    if (a.percol) {
      float gv[VEC];
      if (a.gamma) {
        load_param_vec<VEC>(a.gamma + col, gv);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) gv[j] = 1.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = dv[j] * gv[j] * istd + ca * (xv[j] - mean) + cb;
    } else {
      const uint32_t pidx = (row % a.pmod) * a.pmul + a.pdiv.div(col);
      const float gi = (a.gamma ? a.gamma[pidx] : 1.f) * istd;
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = dv[j] * gi + ca * (xv[j] - mean) + cb;
    }
    if (a.accum_dx) {
      float old[VEC];
      load_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] += old[j];
    }
    store_vec<T, VEC>(dx + static_cast<size_t>(i) * VEC, o);
  }
}

// LayerNormalization dgamma/dbeta partials, any shape.  grid = (ceil(R/(64*VEC)), Y):
// a block owns a strip of 64*VEC columns (a lane VEC adjacent ones: one
// wave-wide, fully coalesced access per row) and the rows [y*rpc, (y+1)*rpc);
// its 4 waves take every 4th row, 4 rows in flight each.
// part[y][0][R] = sum dy*(x-mean)*istd, part[y][1][R] = sum dy;
// ln_param_reduce_kernel folds the Y partials.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
ln_colgrad_stream_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                         const float *__restrict__ mean, const float *__restrict__ var,
                         int rows, int R, int rpc, float eps, float *__restrict__ part) {
  __shared__ float rg[4][64 * VEC];
  __shared__ float rb[4][64 * VEC];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = (blockIdx.x * 64 + lane) * VEC;
  const int colc = col < R ? col : R - VEC; // clamped: loads stay unconditional
  const int rbegin = blockIdx.y * rpc;
  const int rend = min(rbegin + rpc, rows);
  float sg[VEC], sb[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sg[j] = sb[j] = 0.f;
  for (int r0 = rbegin + wave; r0 < rend; r0 += 16) {
    RawVec<T, VEC> xv[4], dv[4];
    float mu[4], is[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int r = r0 + 4 * u;
      const int rc = r < rend ? r : r0;
      const size_t i = static_cast<size_t>(rc) * R + colc;
      xv[u] = load_raw<T, VEC>(x + i);
      dv[u] = raw_or_zero<T, VEC>(r < rend, load_raw<T, VEC>(dy + i));
      mu[u] = mean[rc];
      is[u] = var[rc];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float istd = inv_std(is[u], eps);
      const float nmi = -mu[u] * istd;
      float xf[VEC], df[VEC];
      unpack<T, VEC>(xv[u], xf);
      unpack<T, VEC>(dv[u], df);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        sg[j] = fmaf(df[j], fmaf(xf[j], istd, nmi), sg[j]);
        sb[j] += df[j];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    rg[wave][lane * VEC + j] = sg[j];
    rb[wave][lane * VEC + j] = sb[j];
  }
  lds_barrier();
  if (wave == 0 && col < R) {
    float *p = part + static_cast<size_t>(blockIdx.y) * 2 * R;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int l = lane * VEC + j;
      p[col + j] = (rg[0][l] + rg[1][l]) + (rg[2][l] + rg[3][l]);
      p[R + col + j] = (rb[0][l] + rb[1][l]) + (rb[2][l] + rb[3][l]);
    }
  }
}

// ---------------------------------------------------------------------------
// Second stage of the LayerNormalization parameter gradients: column sums of
// the per-block partials ws[nparts][2][R] -> dgamma[R], dbeta[R].
// Block = 16 columns x 64 part groups: up to 512 partials are one batch of 8
// independent loads per thread (one memory round trip), a 64-byte run per
// part, and 2R/16 blocks spread the fold over the chip.  The fold order is
// fixed: parts py, py+64, ... per thread, lanes by butterfly, waves in order.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(1024)
ln_param_reduce_kernel(const float *__restrict__ ws, int nparts, int R,
                       float *__restrict__ dgamma, float *__restrict__ dbeta,
                       int accum_g, int accum_b) {
  __shared__ float red[16][16];
  const int cx = threadIdx.x & 15;
  const int py = threadIdx.x >> 4;
  const int wave = threadIdx.x >> 6;
  const int col2 = blockIdx.x * 16 + cx; // column in the [2R] concatenation
  const bool live = col2 < 2 * R;
  const size_t stride = 2 * static_cast<size_t>(R);
  float s = 0.f;
  for (int p0 = py; p0 < nparts; p0 += 64 * 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int p = p0 + 64 * u;
      v[u] = (live && p < nparts) ? ws[static_cast<size_t>(p) * stride + col2] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  s = xor_add<32>(xor_add<16>(s));
  if ((threadIdx.x & 63) < 16) red[wave][cx] = s;
  lds_barrier();
  if (threadIdx.x < 16 && live) {
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) tot += red[i][cx];
    if (col2 < R) {
      if (dgamma) dgamma[col2] = tot + (accum_g ? dgamma[col2] : 0.f);
    } else {
      if (dbeta) dbeta[col2 - R] = tot + (accum_b ? dbeta[col2 - R] : 0.f);
    }
  }
}

// The same fold for long rows (R a multiple of 4, ws 16-byte aligned), where
// the partials are tens of MB: block = 16 lanes x 64 part groups, a lane takes
// four adjacent columns in one 16-byte load, so a part contributes a 256-byte
// run per block instead of a 64-byte one ([2048,16384] half, 256 parts of
// 128 KB: 11.1 -> 6.0 us; [4096,8192] 6.5 -> 4.2), and 2R/64 blocks.  Fixed order as above: parts py,
// py+64, ... per thread, lanes by butterfly, waves in order.
__global__ void __launch_bounds__(1024)
ln_param_reduce_wide_kernel(const float *__restrict__ ws, int nparts, int R,
                            float *__restrict__ dgamma, float *__restrict__ dbeta,
                            int accum_g, int accum_b) {
  __shared__ float red[16][16][4];
  const int cx = threadIdx.x & 15;
  const int py = threadIdx.x >> 4;
  const int wave = threadIdx.x >> 6;
  const int col2 = (blockIdx.x * 16 + cx) * 4; // first of the lane's columns in [2R]
  const bool live = col2 < 2 * R;
  const size_t stride = 2 * static_cast<size_t>(R);
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int p0 = py; p0 < nparts; p0 += 64 * 4) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = p0 + 64 * u;
      v[u] = (live && p < nparts)
                 ? *reinterpret_cast<const float4 *>(ws + static_cast<size_t>(p) * stride + col2)
                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      s[0] += v[u].x;
      s[1] += v[u].y;
      s[2] += v[u].z;
      s[3] += v[u].w;
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) s[j] = xor_add<32>(xor_add<16>(s[j]));
  if ((threadIdx.x & 63) < 16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) red[wave][cx][j] = s[j];
  }
  lds_barrier();
  if (threadIdx.x < 64) {
    const int c = threadIdx.x >> 2, j = threadIdx.x & 3;
    const int col = (blockIdx.x * 16 + c) * 4 + j;
    if (col < 2 * R) {
      float tot = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) tot += red[i][c][j];
      if (col < R) {
        if (dgamma) dgamma[col] = tot + (accum_g ? dgamma[col] : 0.f);
      } else {
        if (dbeta) dbeta[col - R] = tot + (accum_b ? dbeta[col - R] : 0.f);
      }
    }
  }
}

} // namespace nblahip
