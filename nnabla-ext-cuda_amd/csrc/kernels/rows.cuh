// Row normalizations (LayerNormalization rows, InstanceNormalization planes,
// GroupNormalization groups) with the row cached in registers: x (and dy) cross
// HBM exactly once per direction.
//
// Thread layout: TPR threads share a row (4..32 = several rows per wavefront,
// for rows of a few hundred bytes; 64 = one wavefront, no barrier at all;
// 256 / 1024 = one block per row, LDS cross-wave merge).  Thread t issues NL
// 16-byte loads at element (k*TPR + t)*VEC, k = 0..NL-1, so every load
// instruction of a wave covers 1 KiB of consecutive memory.
//
// Statistics: the row sits in registers, so the mean is an exact-count sum and
// the variance is the centred second moment taken from the same registers
// (one pass over memory, no E[x^2]-E[x]^2 cancellation).
#pragma once

#include "common.cuh"
#include "launch.hpp"

namespace nblahip {

struct RowArgs {
  const void *x;
  const void *dy;     // backward only
  void *out;          // y (forward) or dx (backward, may be null)
  const float *gamma; // may be null
  const float *beta;  // may be null (forward only)
  float *mean;        // forward: written; backward: read
  float *var;
  const float *dmean; // may be null
  const float *dvar;  // may be null
  float *ws;          // backward partials
  int rows;
  int R;
  float eps;
  float inv_R;
  // Parameter index of element (row, col):
  //   percol != 0 : col                                   (LayerNormalization)
  //   percol == 0 : (row % pmod) * pmul + col / pdiv       (Instance / Group)
  // (beta uses pmod_b in place of pmod: InstanceNormalization may broadcast
  // gamma and beta differently.)
  int percol;
  int ahead; // forward, LayerNormalization: the persistent launch whose blocks ask for their next row ahead
  uint32_t pmod;
  uint32_t pmod_b;
  uint32_t pmul;
  FastDiv pdiv;
  int accum_dx;
  // 1.0f delivered at run time: keeps fma(float(half), one, b) a single
  // mixed-precision instruction (see elem_fma).
  float one;
  // Channel-per-block InstanceNormalization backward writes the parameter
  // gradients itself.
  float *dgamma;
  float *dbeta;
  int accum_g;
  int accum_b;
  // GroupNormalization backward: runs (wave-wide loads) per channel and
  // channels per group, and the thread map (see GnSlot).
  int epc;
  int cpg;
  int gn_wpc;      // waves sharing one channel
  int gn_nwc;      // channels the block's waves cover at once (NW / gn_wpc)
  int gn_pv;       // vectors per plane (spatial / VEC)
  uint64_t gn_map; // per load k, 8 bits: (pass over the channels) | (load within the channel) << 4; 0xff unused
  // BatchNormalization rows (STRIDED / kRowBN): row c is the planes (n, c),
  // n = 0..N-1, each `plane.d` contiguous elements, plane_jump = (C-1)*plane.d
  // elements between the end of one and the start of the next.
  FastDiv plane;
  uint32_t plane_jump;
  // ... planes that are no whole number of 128-byte lines share their first and
  // last line with the neighbouring channels' planes: edge_bytes = the plane's
  // size then (else 0), and neighbouring blocks run on the same XCD (per_xcd
  // blocks each; 0: plain order).
  uint32_t edge_bytes;
  uint32_t per_xcd;
  float *rmean; // running statistics, may be null
  float *rvar;
  float decay, unbias;
};

// Offset of element col of a row from the row's first element.  32 bits (a
// tensor has fewer than 2^31 elements): the row base stays a wave-uniform
// 64-bit value and the per-lane part of every address one register.
template <bool STRIDED>
__device__ __forceinline__ uint32_t row_elem_offset(const RowArgs &a, int col) {
  if constexpr (STRIDED) {
    return static_cast<uint32_t>(col) + a.plane.div(static_cast<uint32_t>(col)) * a.plane_jump;
  } else {
    return static_cast<uint32_t>(col);
  }
}

// BatchNormalization rows: block index with neighbouring channels on the same
// XCD (workgroups go to the 8 XCDs round-robin), whose L2 then fetches a line
// two planes share once and merges the partial writes to it.
template <bool STRIDED> __device__ __forceinline__ uint32_t row_block_index(const RowArgs &a) {
  if constexpr (STRIDED) {
    if (a.per_xcd) return (blockIdx.x % 8u) * a.per_xcd + blockIdx.x / 8u;
  }
  return blockIdx.x;
}

// Store of the vector at column col of a row.  BatchNormalization rows whose
// planes share lines with their neighbours write the vectors inside such a
// line with an ordinary store (L2 merges the line's parts; non-temporal
// stores of line pieces go to memory piece by piece).
template <typename T, int VEC, bool STRIDED>
__device__ __forceinline__ void row_store(const RowArgs &a, T *dst, int col, const float (&o)[VEC]) {
  if constexpr (STRIDED) {
    if (a.edge_bytes) {
      const uint32_t w = static_cast<uint32_t>(col) - a.plane.div(static_cast<uint32_t>(col)) * a.plane.d;
      const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
      const uintptr_t first = addr - static_cast<uintptr_t>(w) * sizeof(T);
      const uintptr_t line = addr >> 7;
      if (line < ((first + 127u) >> 7) || line >= ((first + a.edge_bytes) >> 7)) {
        store_vec<T, VEC, false>(dst, o);
        return;
      }
    }
  }
  store_vec<T, VEC>(dst, o);
}

// GroupNormalization backward thread map.  A wave-wide load never crosses a
// channel, so the per-channel sums the parameter gradients need are wave sums.
// The block's NW waves are split into gn_nwc sets of gn_wpc waves; in pass ci a
// set works on channel ci*gn_nwc + set, whose plane its waves cover in runs of
// 64 vectors: load m of wave j of the set is run m*gn_wpc + j of that channel
// (lanes past the plane's end idle).  Channels with small planes therefore
// share a wave's loads over several passes, channels with large planes spread
// over several waves, and the plane only has to be a whole number of vectors.
struct GnSlot {
  uint32_t ch; // channel within the group
  int run;     // index into the block's run sums: ch*epc + run within the channel
  int col;     // first element within the row
  bool ok;     // this lane holds data
  bool live;   // the wave's run exists (its sums are recorded, zeros included)
};

template <int VEC>
__device__ __forceinline__ GnSlot gn_slot(const RowArgs &a, int k, int set, int j, int lane) {
  GnSlot s;
  const uint32_t code = static_cast<uint32_t>(a.gn_map >> (8 * k)) & 0xffu;
  const int ci = code & 15, m = code >> 4;
  s.ch = static_cast<uint32_t>(ci * a.gn_nwc + set);
  const int part = m * a.gn_wpc + j;
  s.live = code != 0xffu && set < a.gn_nwc && static_cast<int>(s.ch) < a.cpg;
  s.ok = s.live && lane < a.gn_pv - part * kWave;
  s.run = static_cast<int>(s.ch) * a.epc + part;
  s.col = (static_cast<int>(s.ch * a.pdiv.d) + part * (kWave * VEC)) + lane * VEC;
  return s;
}

template <int TPR> struct RowBlock {
  static constexpr int kBlock = TPR < 256 ? 256 : TPR;
  static constexpr int kRowsPerBlock = kBlock / TPR;
};

// Backward blocks.  The LayerNormalization backward is persistent and keeps
// per-column accumulators, so its wave-per-row layout packs 8 rows into a
// 512-thread block (256 VGPRs per lane stay available): two blocks per CU,
// few partials to fold afterwards.
template <int TPR, int MODE> struct RowBwdBlock {
  static constexpr int kBlock = (MODE == kRowLN && TPR <= kWave)    ? 512
                                : (MODE == kRowINc && TPR == kWave) ? 1024
                                                                    : RowBlock<TPR>::kBlock;
  static constexpr int kRowsPerBlock = kBlock / TPR;
};

// Waves per SIMD the backward kernel must leave room for (second argument of
// __launch_bounds__).  Two 512-thread blocks per CU need 4, i.e. at most 128
// VGPRs; the layout named here would otherwise take a few registers more,
// halve its occupancy and run a grid of two blocks per CU in two rounds
// (GroupNormalization backward of 64 KB half groups: 21.5 -> 17.1 us; the
// float layout would spill 96 bytes per lane under the cap and is slower with
// it: 22.4 vs 21.0 us on 16 384-element groups).  The
// wave-per-row LayerNormalization float kernel (133 VGPRs) is left alone: the
// spill the cap costs it sits in its row loop and is worth more than the
// occupancy.
template <typename T, int VEC, int NL, int TPR, int MODE> struct RowBwdOccupancy {
  static constexpr bool kGn512 =
      (MODE == kRowGN || MODE == kRowGNm) && TPR == 512 && NL == 8 && sizeof(T) == 2;
  static constexpr int kMinWaves = kGn512 ? 4 : 1;
};

// ---------------------------------------------------------------------------
// Forward: y, mean, var.  PERCOL selects the LayerNormalization parameter
// layout (gamma/beta per column: loaded once per thread, before the row loop,
// and kept in registers); otherwise one scalar gamma/beta per 16-byte load,
// fetched while the row is still in flight.
// ---------------------------------------------------------------------------
// STRIDED: BatchNormalization rows (see RowArgs::plane); also updates the
// running statistics.
// AHEAD: for a persistent launch (a few blocks per CU, each walking many
// rows): the next row's loads are issued before the current row's sums, so a
// block always has a row in flight.
template <typename T, int VEC, int NL, int TPR, bool PERCOL, bool STRIDED = false, bool AHEAD = false>
__global__ void __launch_bounds__(RowBlock<TPR>::kBlock,
                                  ((PERCOL && TPR == 1024 && NL <= 4) ? 8 : 1))
row_fwd_kernel(const RowArgs a) {
  static_assert(!AHEAD || (PERCOL && !STRIDED), "rows ahead: LayerNormalization only");
  constexpr int RPB = RowBlock<TPR>::kRowsPerBlock;
  __shared__ float lds[2 * 16];
  const int t = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  T *__restrict__ y = static_cast<T *>(a.out);

  // 1024-thread blocks (rows of thousands of vectors, one row per block): the
  // parameters are fetched where they are used instead, which keeps the kernel
  // at 64 VGPRs and two blocks per CU.
  constexpr bool LATE = PERCOL && TPR == 1024;
  float gcol[(PERCOL && !LATE) ? NL : 1][VEC], bcol[(PERCOL && !LATE) ? NL : 1][VEC];
  if constexpr (PERCOL && !LATE) {
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int col = (k * TPR + t) * VEC;
      const bool ok = col < a.R;
      if (ok && a.gamma) {
        load_param_vec<VEC>(a.gamma + col, gcol[k]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) gcol[k][j] = 1.f;
      }
      if (ok && a.beta) {
        load_param_vec<VEC>(a.beta + col, bcol[k]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) bcol[k][j] = 0.f;
      }
    }
  }

  RawVec<T, VEC> ahead[AHEAD ? NL : 1];
  if constexpr (AHEAD) {
    const int row0 = min(static_cast<int>(row_block_index<STRIDED>(a) * RPB + sub), static_cast<int>(a.rows) - 1);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int col = (k * TPR + t) * VEC;
      ahead[k] = load_raw<T, VEC>(x + static_cast<size_t>(row0) * a.R + (col < a.R ? col : 0));
    }
  }
  for (int row = row_block_index<STRIDED>(a) * RPB + sub; row < a.rows; row += gridDim.x * RPB) {
    const size_t base = static_cast<size_t>(row) * (STRIDED ? a.plane.d : a.R);
    RawVec<T, VEC> raw[NL];
    if constexpr (AHEAD) {
      // (behind the last row: that row again - a load nobody waits for)
      const int nrow = min(row + static_cast<int>(gridDim.x) * RPB, static_cast<int>(a.rows) - 1);
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const int col = (k * TPR + t) * VEC;
        raw[k] = raw_or_zero<T, VEC>(col < a.R, ahead[k]);
        ahead[k] = load_raw<T, VEC>(x + static_cast<size_t>(nrow) * a.R + (col < a.R ? col : 0));
      }
    } else {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        // Out-of-row lanes load column 0 (always valid) and are zeroed after:
        // no branch, so the NL loads are in flight together.
        const int col = (k * TPR + t) * VEC;
        const bool ok = col < a.R;
        raw[k] = raw_or_zero<T, VEC>(
            ok, load_raw<T, VEC>(x + base + row_elem_offset<STRIDED>(a, ok ? col : 0)));
      }
    }
    float gk[PERCOL ? 1 : NL], bk[PERCOL ? 1 : NL];
    if constexpr (!PERCOL) {
      const uint32_t pbase = (static_cast<uint32_t>(row) % a.pmod) * a.pmul;
      const uint32_t bbase = (static_cast<uint32_t>(row) % a.pmod_b) * a.pmul;
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const int col = (k * TPR + t) * VEC;
        const uint32_t poff = (col < a.R) ? a.pdiv.div(static_cast<uint32_t>(col)) : 0u;
        gk[k] = a.gamma ? a.gamma[pbase + poff] : 1.f;
        bk[k] = a.beta ? a.beta[bbase + poff] : 0.f;
      }
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
      const int col = (k * TPR + t) * VEC;
      if (col < a.R) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = elem_fma<T, VEC>(raw[k], j, a.one, -mean);
          q = fmaf(d, d, q);
        }
      }
    }
    const float var = row_sum<TPR>(q, lds) * a.inv_R;
    const float istd = inv_std(var, a.eps);
    if (t == 0) {
      a.mean[row] = mean;
      a.var[row] = var;
      if constexpr (STRIDED) {
        if (a.rmean) a.rmean[row] = a.decay * a.rmean[row] + (1.f - a.decay) * mean;
        if (a.rvar) a.rvar[row] = a.decay * a.rvar[row] + (1.f - a.decay) * var * a.unbias;
      }
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) keep_packed<T, VEC>(raw[k]);

#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int col = (k * TPR + t) * VEC;
      if (col < a.R) {
        float o[VEC];
        if constexpr (LATE) {
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
          for (int j = 0; j < VEC; ++j)
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), gv[j] * istd, bv[j]);
        } else if constexpr (PERCOL) {
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), gcol[k][j] * istd, bcol[k][j]);
        } else if constexpr (sizeof(T) == 2) {
          // Half output: x*g + (b - mean*g) in one mixed fma per element; the
          // folded shift loses nothing a 10-bit mantissa can hold.
          const float g = gk[k] * istd;
          const float sh = fmaf(-mean, g, bk[k]);
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = elem_fma<T, VEC>(raw[k], j, g, sh);
        } else {
          const float g = gk[k] * istd;
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            o[j] = fmaf(elem_fma<T, VEC>(raw[k], j, a.one, -mean), g, bk[k]);
        }
        row_store<T, VEC, (STRIDED && TPR * NL < 8192)>(a, y + base + row_elem_offset<STRIDED>(a, col), col, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Backward: dx plus partial parameter gradients.  With xh = (x-mean)*istd
// (one fma per element: x*istd - mean*istd) and dg = dy*gamma:
//   s1 = sum(dg), t2 = sum(dg*xh)
//   cA = -istd*t2/R + 2*dvar*std/R        cb = -s1*istd/R + dmean/R
//   dx = dg*istd + cA*xh + cb
// which is the reference's a*x+b form (kernel/layer_normalization.cuh:50-95)
// rewritten on the normalised variable (std = (var+eps)*istd).
//
// Partial parameter gradients written to ws:
//   LN : ws[block][0][R] = sum_rows dy*xh, ws[block][1][R] = sum_rows dy
//   IN : ws[2*row] = sum dy*xh, ws[2*row+1] = sum dy             (row = (n,c))
//   GN : same pair per (n, channel); every wave-wide load lies inside one
//        channel, by the fixed map when spatial % (64*VEC) == 0 (kRowGN), else by
//        the run-time map of GnSlot (kRowGNm).
// Padded lanes hold x = dy = 0 in registers; dy == 0 keeps them out of every
// sum.
// ---------------------------------------------------------------------------
// BAHEAD (LayerNormalization): the block asks for its next row's x, dy and
// statistics before it works on the current row.
template <typename T, int VEC, int NL, int TPR, int MODE, bool BAHEAD = false>
__global__ void __launch_bounds__((RowBwdBlock<TPR, MODE>::kBlock),
                                   (RowBwdOccupancy<T, VEC, NL, TPR, MODE>::kMinWaves))
row_bwd_kernel(const RowArgs a) {
  static_assert(!BAHEAD || MODE == kRowLN, "rows ahead: LayerNormalization only");
  constexpr int RPB = RowBwdBlock<TPR, MODE>::kRowsPerBlock;
  constexpr int NW = TPR / kWave;
  // LayerNormalization keeps xh and dg of a row in registers between the
  // reduction and the dx step when they are few; otherwise they are recomputed.
  // (not with the next row's vectors in registers as well)
  constexpr bool KEEP = (MODE == kRowLN) && (NL * VEC <= 16) && !BAHEAD;
  constexpr bool GN = MODE == kRowGN || MODE == kRowGNm;
  constexpr bool BN = MODE == kRowBN; // strided rows, dgamma/dbeta written here
  constexpr bool GNM = MODE == kRowGNm; // run-time thread map (GnSlot)
  // Float groups of 64-128 KB (1024 threads x 8 loads): dy waits in LDS, not
  // in registers (each thread reads back what it wrote) - with x and dy both
  // in registers the block is alone on its CU at 128 registers per thread and
  // loses to the five-pass streaming kernels.
  constexpr bool PARK = GN && sizeof(T) == 4 && VEC == 4 && TPR == 1024 && NL == 8;
  __shared__ uint4 park[PARK ? NL * TPR : 1];
  __shared__ float lds[2 * 16];
  __shared__ float part[GN ? 2 * NW * NL : 1];
  __shared__ float xfold[(MODE == kRowLN && RPB > 1) ? 2 * NL * (RPB / 2) * TPR * VEC : 1];
  const int t = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const T *__restrict__ x = static_cast<const T *>(a.x);
  const T *__restrict__ dy = static_cast<const T *>(a.dy);
  T *__restrict__ dx = static_cast<T *>(a.out);

  float acc_g[(MODE == kRowLN) ? NL : 1][VEC];
  float acc_b[(MODE == kRowLN) ? NL : 1][VEC];
  float gcol[(MODE == kRowLN) ? NL : 1][VEC]; // per-column gamma, loaded once
  if constexpr (MODE == kRowLN) {
#pragma unroll
    for (int k = 0; k < NL; ++k) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc_g[k][j] = acc_b[k][j] = 0.f;
      const int col = (k * TPR + t) * VEC;
      if (col < a.R && a.gamma) {
        load_param_vec<VEC>(a.gamma + col, gcol[k]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) gcol[k][j] = 1.f;
      }
    }
  }

  // GroupNormalization: this wave's set, its place within the set, the lane.
  int gn_set = 0, gn_j = 0, gn_lane = 0;
  if constexpr (GNM) {
    // wave-uniform, and told so: the map then costs scalar instructions only
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / kWave));
    gn_set = wave / a.gn_wpc;
    gn_j = wave - gn_set * a.gn_wpc;
    gn_lane = threadIdx.x & (kWave - 1);
  }

  // Iteration space.  Every mode but kRowINc: one unit = one row, rows strided
  // over the grid.  kRowINc: one unit = one channel (block-strided), whose
  // batch*1 rows (n, c) are strided over the block's waves / walked in turn.
  constexpr bool CH = (MODE == kRowINc);
  const int channels = static_cast<int>(a.pmod);
  const int nunits = CH ? channels : a.rows;
  const int u0 = CH ? static_cast<int>(blockIdx.x) : static_cast<int>(row_block_index<BN>(a)) * RPB + sub;
  const int ustride = CH ? static_cast<int>(gridDim.x) : static_cast<int>(gridDim.x) * RPB;
  const int inner_n = CH ? a.rows / channels : 1;
  RawVec<T, VEC> xa[BAHEAD ? NL : 1], da[BAHEAD ? NL : 1];
  float mean_a = 0.f, var_a = 0.f;
  if constexpr (BAHEAD) {
    const int r0 = min(u0, nunits - 1);
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int col = (k * TPR + t) * VEC;
      const size_t o = static_cast<size_t>(r0) * a.R + (col < a.R ? col : 0);
      xa[k] = load_raw<T, VEC>(x + o);
      da[k] = load_raw<T, VEC>(dy + o);
    }
    mean_a = a.mean[r0];
    var_a = a.var[r0];
  }
  for (int unit = u0; unit < nunits; unit += ustride) {
  float ch_sdx = 0.f, ch_sdy = 0.f; // kRowINc: this wave's share of the channel sums
  for (int rr = CH ? sub : 0; rr < inner_n; rr += CH ? RPB : 1) {
    const int row = CH ? rr * channels + unit : unit;
    const size_t base = static_cast<size_t>(row) * (BN ? a.plane.d : a.R);
    float gk[NL];                                   // per-load scalar gamma (IN / GN)
    float gch = 1.f;                                // GN: gamma of channel threadIdx.x
    if constexpr (GN) {
      // Issued ahead of the row data, so their latency hides behind it.
      const uint32_t pb = (static_cast<uint32_t>(row) % a.pmod) * a.pmul;
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        if constexpr (GNM) {
          const GnSlot sl = gn_slot<VEC>(a, k, gn_set, gn_j, gn_lane);
          gk[k] = (a.gamma && sl.live) ? a.gamma[pb + sl.ch] : 1.f;
        } else {
          const int col = (k * TPR + t) * VEC;
          const uint32_t ch = (col < a.R) ? a.pdiv.div(static_cast<uint32_t>(col)) : 0u;
          gk[k] = a.gamma ? a.gamma[pb + ch] : 1.f;
        }
      }
      if (a.gamma && static_cast<int>(threadIdx.x) < a.cpg) gch = a.gamma[pb + threadIdx.x];
    }
    // IN: the row's gamma, asked for ahead of the row (behind the reduction it
    // would cost a memory round trip of its own; the BN rows have no register
    // to spare for it).
    float g_row = 1.f;
    if constexpr (MODE == kRowIN || MODE == kRowINc) {
      if (a.gamma) g_row = a.gamma[(static_cast<uint32_t>(row) % a.pmod) * a.pmul];
    }
    // (with dy parked in LDS the statistics too: the stores wait for the row)
    float mean_early = 0.f, var_early = 0.f;
    if constexpr (PARK) {
      mean_early = a.mean[row];
      var_early = a.var[row];
    }
    RawVec<T, VEC> xr[NL], dr[NL];
    float mean_now = 0.f, var_now = 0.f;
    if constexpr (BAHEAD) {
      // (behind the block's last row: the tensor's last row again - loads nobody waits for)
      const int nrow = min(unit + ustride, nunits - 1);
      mean_now = mean_a;
      var_now = var_a;
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const int col = (k * TPR + t) * VEC;
        const bool ok = col < a.R;
        xr[k] = raw_or_zero<T, VEC>(ok, xa[k]);
        dr[k] = raw_or_zero<T, VEC>(ok, da[k]);
        const size_t o = static_cast<size_t>(nrow) * a.R + (ok ? col : 0);
        xa[k] = load_raw<T, VEC>(x + o);
        da[k] = load_raw<T, VEC>(dy + o);
      }
      mean_a = a.mean[nrow];
      var_a = a.var[nrow];
    } else
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      int col = (k * TPR + t) * VEC;
      bool ok = col < a.R;
      if constexpr (GNM) {
        const GnSlot sl = gn_slot<VEC>(a, k, gn_set, gn_j, gn_lane);
        col = sl.col;
        ok = sl.ok;
      }
      // branch-free: all loads in flight together
      const uint32_t off = row_elem_offset<BN>(a, ok ? col : 0);
      xr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(x + base + off));
      dr[k] = raw_or_zero<T, VEC>(ok, load_raw<T, VEC>(dy + base + off));
    }
    if constexpr (PARK) {
#pragma unroll
      for (int k = 0; k < NL; ++k) park[k * TPR + threadIdx.x] = __builtin_bit_cast(uint4, dr[k]);
      asm volatile("" ::: "memory"); // read back from LDS from here on
    }
    auto dyv = [&](int k) -> RawVec<T, VEC> {
      if constexpr (PARK) {
        return __builtin_bit_cast(RawVec<T, VEC>, park[k * TPR + threadIdx.x]);
      } else {
        return dr[k];
      }
    };
    const float mean = BAHEAD ? mean_now : PARK ? mean_early : a.mean[row];
    const float vpe = (BAHEAD ? var_now : PARK ? var_early : a.var[row]) + a.eps;
    const float istd = 1.0f / sqrtf(vpe);
    const float nmi = -mean * istd;

    float s1 = 0.f, t2 = 0.f;
    float xh_keep[KEEP ? NL : 1][VEC], dg_keep[KEEP ? NL : 1][VEC];
    if constexpr (MODE == kRowLN) {
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
    } else if constexpr (MODE == kRowLNx) {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const int col = (k * TPR + t) * VEC;
        float gv[VEC];
        if (col < a.R && a.gamma) {
          load_param_vec<VEC>(a.gamma + col, gv);
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) gv[j] = 1.f;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          const float dg = elem_fma<T, VEC>(dr[k], j, gv[j], 0.f);
          s1 += dg;
          t2 = fmaf(dg, xh, t2);
        }
      }
      row_sum2<TPR>(s1, t2, lds);
    } else if constexpr (MODE == kRowIN || MODE == kRowINc || BN) {
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
      if constexpr (CH) {
        ch_sdx += sdx;
        ch_sdy += sdy;
      } else if constexpr (BN) {
        if (t == 0) {
          if (a.dgamma) a.dgamma[row] = sdx + (a.accum_g ? a.dgamma[row] : 0.f);
          if (a.dbeta) a.dbeta[row] = sdy + (a.accum_b ? a.dbeta[row] : 0.f);
        }
      } else {
        if (t == 0) {
          a.ws[2 * static_cast<size_t>(row)] = sdx;
          a.ws[2 * static_cast<size_t>(row) + 1] = sdy;
        }
      }
      float g = g_row;
      if constexpr (BN) g = a.gamma ? a.gamma[(static_cast<uint32_t>(row) % a.pmod) * a.pmul] : 1.f;
#pragma unroll
      for (int k = 0; k < NL; ++k) gk[k] = g;
      s1 = g * sdy;
      t2 = g * sdx;
    } else { // GroupNormalization, RPB == 1
      static_assert(!GN || RPB == 1, "group rows own the whole block");
      const int lane = threadIdx.x & (kWave - 1);
      const uint32_t pbase = (static_cast<uint32_t>(row) % a.pmod) * a.pmul;
      lds_barrier(); // part[] of the previous row has been consumed
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        const RawVec<T, VEC> dk = dyv(k);
        float sdy = raw_sum<T, VEC>(dk, 0.f);
        float sdx = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
          sdx = elem_fma<T, VEC>(dk, j, xh, sdx);
        }
        sdy = wave_sum(sdy);
        sdx = wave_sum(sdx);
        if constexpr (GNM) {
          const GnSlot sl = gn_slot<VEC>(a, k, gn_set, gn_j, gn_lane);
          if (lane == 0 && sl.live) {
            part[2 * sl.run] = sdx;
            part[2 * sl.run + 1] = sdy;
          }
        } else {
          // fixed map: run e covers elements [e*64*VEC, (e+1)*64*VEC) of the row
          const int e = k * NW + static_cast<int>(threadIdx.x / kWave);
          if (lane == 0) {
            part[2 * e] = sdx;
            part[2 * e + 1] = sdy;
          }
        }
      }
      lds_barrier();
      // Channel c owns runs [c*epc, (c+1)*epc).
      float c1 = 0.f, c2 = 0.f;
      for (int c = threadIdx.x; c < a.cpg; c += TPR) {
        float sdx = 0.f, sdy = 0.f;
        for (int e = c * a.epc; e < (c + 1) * a.epc; ++e) {
          sdx += part[2 * e];
          sdy += part[2 * e + 1];
        }
        const size_t o = 2 * (static_cast<size_t>(row) * a.cpg + c);
        a.ws[o] = sdx;
        a.ws[o + 1] = sdy;
        const float g = c < TPR ? gch : (a.gamma ? a.gamma[pbase + c] : 1.f);
        c1 += g * sdy;
        c2 += g * sdx;
      }
      row_sum2<TPR>(c1, c2, lds);
      s1 = c1;
      t2 = c2;
    }

#pragma unroll
    for (int k = 0; k < NL; ++k) {
      keep_packed<T, VEC>(xr[k]);
      if constexpr (!PARK) keep_packed<T, VEC>(dr[k]);
    }
    const float cA = -istd * t2 * a.inv_R +
                     (a.dvar ? 2.f * a.dvar[row] * (vpe * istd) * a.inv_R : 0.f);
    const float cb = -s1 * istd * a.inv_R + (a.dmean ? a.dmean[row] * a.inv_R : 0.f);

    if (dx != nullptr) {
#pragma unroll
      for (int k = 0; k < NL; ++k) {
        int col = (k * TPR + t) * VEC;
        bool ok = col < a.R;
        if constexpr (GNM) {
          const GnSlot sl = gn_slot<VEC>(a, k, gn_set, gn_j, gn_lane);
          col = sl.col;
          ok = sl.ok;
        }
        if (ok) {
          float o[VEC];
          if constexpr (KEEP) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              o[j] = fmaf(dg_keep[k][j], istd, fmaf(xh_keep[k][j], cA, cb));
          } else if constexpr (MODE == kRowLN) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
              o[j] = elem_fma<T, VEC>(dr[k], j, gcol[k][j] * istd, fmaf(xh, cA, cb));
            }
          } else if constexpr (MODE == kRowLNx) {
            float gv[VEC]; // read again rather than kept: NL*VEC registers otherwise
            if (a.gamma) {
              load_param_vec<VEC>(a.gamma + col, gv);
            } else {
#pragma unroll
              for (int j = 0; j < VEC; ++j) gv[j] = 1.f;
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
              o[j] = elem_fma<T, VEC>(dr[k], j, gv[j] * istd, fmaf(xh, cA, cb));
            }
          } else {
            const float gi = gk[k] * istd;
            const RawVec<T, VEC> dk = dyv(k);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float xh = norm_elem<T, VEC>(xr[k], j, mean, istd, nmi);
              o[j] = elem_fma<T, VEC>(dk, j, gi, fmaf(xh, cA, cb));
            }
          }
          T *dst = dx + base + row_elem_offset<BN>(a, col);
          if (a.accum_dx) {
            float old[VEC];
            load_vec<T, VEC>(dst, old);
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] += old[j];
          }
          row_store<T, VEC, (BN && TPR * NL < 8192)>(a, dst, col, o);
        }
      }
    }
  } // rows of the unit
  if constexpr (CH) {
    // Fold the waves' shares in wave order and publish dgamma[c], dbeta[c].
    __shared__ float chfold[2 * 16];
    if constexpr (RPB > 1) {
      lds_barrier();
      if (t == 0) {
        chfold[2 * sub] = ch_sdx;
        chfold[2 * sub + 1] = ch_sdy;
      }
      lds_barrier();
      ch_sdx = 0.f;
      ch_sdy = 0.f;
#pragma unroll
      for (int w = 0; w < RPB; ++w) {
        ch_sdx += chfold[2 * w];
        ch_sdy += chfold[2 * w + 1];
      }
    }
    if (threadIdx.x == 0) {
      if (a.dgamma) a.dgamma[unit] = ch_sdx + (a.accum_g ? a.dgamma[unit] : 0.f);
      if (a.dbeta) a.dbeta[unit] = ch_sdy + (a.accum_b ? a.dbeta[unit] : 0.f);
    }
  }
  } // units

  if constexpr (MODE == kRowLN) {
    // Fold the RPB row groups of a block into group 0 (a halving tree, fixed
    // order; every accumulator of a thread goes through a level together: two
    // barriers per level, not two per level and accumulator), then write the
    // block's partial [2][R].
    float *wsb = a.ws + static_cast<size_t>(blockIdx.x) * 2 * a.R;
    if constexpr (RPB > 1) {
      constexpr int kSlab = (RPB / 2) * TPR * VEC; // one accumulator of every thread of the upper half
#pragma unroll
      for (int half = RPB / 2; half >= 1; half /= 2) {
        lds_barrier(); // the previous level has been read
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
        const int col = (k * TPR + t) * VEC;
        if (col < a.R) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) wsb[col + j] = acc_g[k][j];
#pragma unroll
          for (int j = 0; j < VEC; ++j) wsb[static_cast<size_t>(a.R) + col + j] = acc_b[k][j];
        }
      }
    }
  }
}

} // namespace nblahip
