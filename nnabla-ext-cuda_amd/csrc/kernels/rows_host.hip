// Plan selection and launch sequences for the row normalizations
// (LayerNormalization, InstanceNormalization, GroupNormalization), plus the
// instantiations of the streaming kernels.
#include <algorithm>

#include "rows_dispatch.hpp"
#include "pair_reduce.cuh"
#include "rows_stream.cuh"

namespace nblahip {

// max_nl bounds the loads per thread of the layouts below 1024 threads,
// max_nl_1024 those of the 1024-thread layout, whose register budget is 128
// VGPRs; both are chosen per kernel family so that no variant in use spills.
// Rows of fewer than 64 vectors: several rows per wave, 4 to 32 lanes each.
// Measured on 64 MB tensors (LayerNormalization of 32- to 256-element half
// rows: 219 / 106 / 56 / 31 us with a wave per row, 23 / 22 / 22 / 21 us here):
// layouts that pad the row to the next power of two and no further are
// equivalent within 5 %, two loads per lane being the best or next to it in
// both directions; rows of 33 to 63 vectors (7x7 planes) want four loads per
// lane in the forward pass (12.5 vs 18.3 us), which the LayerNormalization
// backward cannot afford in registers.
static bool pick_subwave(RowCfg &c, int64_t nv, bool percol) {
  const int ftpr = tune_int("ROW_TPR", 0), fnl = tune_int("ROW_NL", 0);
  auto take = [&](int tpr, int nl) {
    c.ok = true;
    c.tpr = tpr;
    c.nl = nl;
    return true;
  };
  if (ftpr > 0 && ftpr < 64 && fnl > 0 && static_cast<int64_t>(ftpr) * fnl >= nv)
    return take(ftpr, fnl);
  if (nv >= 64 || !tune_int("ROW_SUBWAVE", 1)) return false;
  if (nv <= 4) return take(4, 1);
  int pad = 8;
  while (pad < nv) pad <<= 1;
  if (pad < 64) return take(pad / 2, 2);
  return percol ? take(32, 2) : take(16, 4);
}

RowCfg pick_row_cfg(int vec, int64_t R, int max_nl, int max_nl_1024, int min_tpr, bool percol,
                    bool three) {
  RowCfg c;
  c.vec = vec;
  const int64_t nv = R / c.vec;
  if (min_tpr < 64 && pick_subwave(c, nv, percol)) return c;
  static const int tprs[4] = {64, 256, 512, 1024};
  static const int nls[5] = {1, 2, 3, 4, 8};
  // (for sweeps: a layout of whole waves forced where it holds the row)
  if (const int ftpr = tune_int("ROW_TPR", 0), fnl = tune_int("ROW_NL", 0);
      ftpr >= 64 && ftpr >= min_tpr && fnl > 0 && static_cast<int64_t>(ftpr) * fnl >= nv) {
    for (int tpr : tprs)
      for (int nl : nls)
        if (tpr == ftpr && nl == fnl && nl <= (tpr == 1024 ? max_nl_1024 : max_nl) && (nl != 3 || three)) {
          c.ok = true;
          c.tpr = tpr;
          c.nl = nl;
          return c;
        }
  }
  for (int tpr : tprs) {
    if (tpr < min_tpr) continue;
    const int cap = tpr == 1024 ? max_nl_1024 : max_nl;
    for (int nl : nls) {
      if (nl > cap) break;
      if (nl == 3 && !three) continue;
      if (static_cast<int64_t>(tpr) * nl >= nv) {
        c.ok = true;
        c.tpr = tpr;
        c.nl = nl;
        return c;
      }
    }
  }
  return c;
}

// LayerNormalization backward.  Measured on 134 MB tensors: the wave-per-row
// layout wins whenever a row fits it with at most 4 loads per lane; otherwise
// 256 or 512 threads with the fewest loads per thread (the per-column
// accumulators make every load cost about 27 VGPRs), and the 1024-thread
// layout, the slowest, only for rows nothing else holds.
// rows: how many there are (0: unknown); the layouts that ask for the next row
// ahead want several rows per block.
static RowCfg pick_ln_bwd_cfg(int dtype, int64_t R, int vec, bool allow_three = true, int64_t rows = 0) {
  RowCfg c;
  c.vec = vec;
  const int64_t nv = R / c.vec;
  auto take = [&](int tpr, int nl) {
    c.ok = true;
    c.tpr = tpr;
    c.nl = nl;
    return c;
  };
  if (pick_subwave(c, nv, true)) return c;
  const bool three = allow_three && vec == (dtype == NBLAHIP_F16 ? 8 : 4) && tune_int("ROW_NL3", 1);
  // (for sweeps: a layout of 64, 256 or 512 threads forced where it holds the row)
  if (const int ftpr = tune_int("LN_BWD_TPR", 0), fnl = tune_int("LN_BWD_NL", 0);
      (ftpr == 64 || ftpr == 256 || ftpr == 512) && (fnl == 1 || fnl == 2 || fnl == 4 || (fnl == 3 && three)) &&
      static_cast<int64_t>(ftpr) * fnl >= nv)
    return take(ftpr, fnl);
  for (int nl : {1, 2, 3, 4})
    if ((nl != 3 || three) && 64 * nl >= nv) return take(64, nl);
  // Half rows of 257 - 512 vectors: 256 threads with two vectors each and the
  // next row asked for ahead, not 512 threads with one (backward cold, us:
  // [13056,2560] 55.3 -> 47.4, [10752,3072] 49.6 -> 42.4, [8192,4096] 46.9 -> 43.8;
  // without the rows ahead it loses, 59.5 / 53.2 / 50.6; float: 1280 - 2048
  // elements 46.4 / 43.2 / 42.0 with 512 x 1 against 55.0 / 49.6 / 45.9).
  if (dtype == NBLAHIP_F16 && vec == 8 && nv > 256 && nv <= 512 && rows >= 2048 &&
      tune_int("LN_BWD_AHEAD", 1) && tune_int("LN_BWD_256X2", 1))
    return take(256, 2);
  for (int nl : {1, 2, 3, 4})
    for (int tpr : {256, 512})
      if ((nl != 3 || three) && static_cast<int64_t>(tpr) * nl >= nv) return take(tpr, nl);
  const int cap_1024 = dtype == NBLAHIP_F16 ? 1 : 2; // beyond: spills
  for (int nl : {1, 2})
    if (nl <= cap_1024 && 1024 * nl >= nv) return take(1024, nl);
  return c;
}

static bool ln_bwd_rows_ahead(int dtype, const RowCfg &c, int vec) {
  if (dtype == NBLAHIP_F16) return vec == 8 && (c.nl == 2 || c.nl == 3) && (c.tpr == 256 || c.tpr == 512);
  return vec == 4 && c.nl == 3 && c.tpr == 512;
}

// GroupNormalization backward: vector width, block size, loads per thread and
// the thread map of GnSlot (written into a).  Candidates are the widest vector
// and scalar loads, and the block sizes whose map fits 8 loads per thread; the
// cost of one is its lane slots (threads x loads) weighted by 4 + VEC: a load
// costs the same whether 8 or 64 of its lanes carry data, but the arithmetic
// behind it grows with the vector, so sparse wide loads lose to dense narrow
// ones (planes of 64 half elements: 15.5 us with 8 of 64 lanes busy, 9.4 us
// with scalar loads).
static RowCfg pick_gn_bwd_cfg(const RowProblem &p, int row_vec, RowArgs &a) {
  RowCfg best;
  const int64_t cpg = p.channels / p.groups;
  int64_t best_cost = 0;
  for (int vec : {row_vec, 1}) {
    const int64_t pv = p.spatial / vec;
    for (int tpr : {256, 512, 1024}) {
      const int64_t nw = tpr / 64;
      const int64_t wpc = cpg < nw ? nw / cpg : 1;
      const int64_t nwc = nw / wpc;
      const int64_t cpw = (cpg + nwc - 1) / nwc;            // passes over the channels
      const int64_t nlc = (pv + 64 * wpc - 1) / (64 * wpc); // loads per channel
      const int64_t need = cpw * nlc;
      if (need > 8 || nlc > 15 || cpw > 15) continue;
      int nl = 1;
      while (nl < need) nl <<= 1;
      const int64_t cost = static_cast<int64_t>(tpr) * nl * (4 + vec);
      if (best.ok && cost >= best_cost) continue;
      best.ok = true;
      best.vec = vec;
      best.tpr = tpr;
      best.nl = nl;
      best_cost = cost;
      a.gn_wpc = static_cast<int>(wpc);
      a.gn_nwc = static_cast<int>(nwc);
      a.gn_pv = static_cast<int>(pv);
      a.epc = static_cast<int>(nlc * wpc);
      uint64_t map = ~0ull;
      for (int64_t k = 0; k < need; ++k) {
        const uint64_t code = static_cast<uint64_t>(k / nlc) | (static_cast<uint64_t>(k % nlc) << 4);
        map = (map & ~(0xffull << (8 * k))) | (code << (8 * k));
      }
      a.gn_map = map;
    }
  }
  return best;
}

static int rows_per_block(int tpr) { return tpr < 256 ? 256 / tpr : 1; }

static int cached_grid(int64_t rows, int tpr) {
  const int rpb = rows_per_block(tpr);
  const int64_t blocks = (rows + rpb - 1) / rpb;
  return static_cast<int>(std::min<int64_t>(blocks, 1 << 20));
}

// Persistent grid of the LayerNormalization backward: each block keeps
// per-column accumulators, so fewer blocks mean fewer partials to fold.
static int ln_bwd_grid(int64_t rows, int tpr, int resident = 2) {
  // Wave-per-row rows run 8 to a 512-thread block; longer rows own a block.
  // resident: blocks of the chosen kernel that fit a CU together; the grid
  // never exceeds what is resident (one round) nor two blocks per CU (the
  // workspace holds one partial per block).
  const int rpb = tpr <= 64 ? 512 / tpr : 1;
  const int per_cu = tune_int("LN_BWD_BLOCKS_PER_CU", std::max(1, std::min(2, resident)));
  const int64_t cap = static_cast<int64_t>(device_cus()) * per_cu;
  const int64_t blocks = (rows + rpb - 1) / rpb;
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(blocks, cap)));
}

static int stream_grid(int64_t work_blocks) {
  const int64_t cap = static_cast<int64_t>(device_cus()) * 16;
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(work_blocks, cap)));
}

static RowArgs make_args(const RowProblem &p) {
  RowArgs a{};
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
  a.eps = p.eps;
  a.inv_R = 1.0f / static_cast<float>(p.R);
  a.accum_dx = p.accum_dx;
  a.dgamma = p.dgamma;
  a.dbeta = p.dbeta;
  a.accum_g = p.accum_g;
  a.accum_b = p.accum_b;
  a.one = 1.0f;
  a.epc = 0;
  a.cpg = 1;
  if (p.mode == kRowLN) {
    a.percol = 1;
    a.pmod = a.pmod_b = 1;
    a.pmul = 0;
    a.pdiv = FastDiv(1);
  } else if (p.mode == kRowIN) {
    a.percol = 0;
    a.pmod = static_cast<uint32_t>(p.bc_gamma ? p.channels : p.rows);
    a.pmod_b = static_cast<uint32_t>(p.bc_beta ? p.channels : p.rows);
    a.pmul = 1;
    a.pdiv = FastDiv(static_cast<uint32_t>(p.R)); // col / R == 0
  } else {
    a.percol = 0;
    a.pmod = a.pmod_b = static_cast<uint32_t>(p.groups);
    a.pmul = static_cast<uint32_t>(p.channels / p.groups);
    a.pdiv = FastDiv(static_cast<uint32_t>(p.spatial));
    a.cpg = static_cast<int>(p.channels / p.groups);
  }
  return a;
}

// Vector width of the row kernels: rows (and GroupNormalization planes) must
// be a whole number of vectors and every pointer 16-byte aligned; 16 bytes, or
// 8 bytes for half rows of 4k elements, else scalar.
static int row_vec(const RowProblem &p, bool backward) {
  if (!aligned16(p.x)) return 1;
  if (p.out && !aligned16(p.out)) return 1;
  if (backward && !aligned16(p.dy)) return 1;
  if (p.mode == kRowLN) {
    if (p.gamma && !aligned16(p.gamma)) return 1;
    if (!backward && p.beta && !aligned16(p.beta)) return 1;
  }
  const int full = p.dtype == NBLAHIP_F16 ? 8 : 4;
  for (int vec : {full, 4}) {
    if (p.R % vec != 0) continue;
    if (p.mode == kRowGN && p.spatial % vec != 0) continue;
    return vec;
  }
  return 1;
}

// Splits per row (or plane) of the streaming reductions: 1 when the units
// alone give every CU two blocks, else enough runs for four blocks per CU, each
// at least four unrolled steps long, at most 64.
static int stream_splits(int64_t units, int64_t nv) {
  const int64_t cus = device_cus();
  if (units >= 2 * cus) return 1;
  const int64_t want = (4 * cus + units - 1) / units;
  const int64_t most = std::max<int64_t>(1, nv / (kStreamBlock * 16));
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(std::min(want, most), 64)));
}

template <typename T, int VEC>
static int stream_fwd_t(const RowProblem &p, const RowArgs &a, hipStream_t st) {
  // A few very long rows: split them.  The partial states live in the first
  // bytes of y, which the apply step below overwrites (not when y is x).
  int S = (p.out != p.x && aligned16(p.out)) ? stream_splits(p.rows, p.R / VEC) : 1;
  float *part = static_cast<float *>(p.out);
  if (static_cast<size_t>(p.rows) * S * 3 * sizeof(float) >
      static_cast<size_t>(p.rows) * p.R * sizeof(T))
    S = 1;
  NBLAHIP_LAUNCH("row_stats_stream_kernel", (row_stats_stream_kernel<T, VEC>),
                 dim3(stream_grid(p.rows), S), dim3(kStreamBlock), 0, st,
                 static_cast<const T *>(p.x), a.rows, a.R, a.inv_R, p.mean, p.var, part);
  if (int e = last_launch_status()) return e;
  if (S > 1) {
    NBLAHIP_LAUNCH("row_stats_merge_kernel", row_stats_merge_kernel, dim3((a.rows + 63) / 64),
                   dim3(64), 0, st, part, a.rows, S, a.inv_R, p.mean, p.var);
    if (int e = last_launch_status()) return e;
  }
  const uint32_t total_vec = static_cast<uint32_t>(p.rows * p.R / VEC);
  NBLAHIP_LAUNCH("row_apply_fwd_kernel", (row_apply_fwd_kernel<T, VEC>), dim3(stream_grid((total_vec + 255) / 256)),
                     dim3(256), 0, st, a, FastDiv(static_cast<uint32_t>(p.R / VEC)), total_vec);
  return last_launch_status();
}

int launch_row_fwd(const RowProblem &p, hipStream_t st) {
  if (int status = 0; !tune_int("FORCE_STREAM", 0) && row_masked_fwd(p, st, &status)) return status;
  const int vec = row_vec(p, false);
  const RowArgs a = make_args(p);
  // LayerNormalization keeps gamma/beta of its columns in registers too: with
  // 8 loads per thread it needs 140-210 VGPRs (8 waves per CU), so it spreads
  // a row over more threads instead.
  const int max_nl = p.mode == kRowLN ? 4 : 8;
  const bool three = vec == (p.dtype == NBLAHIP_F16 ? 8 : 4) && tune_int("ROW_NL3", 1);
  const RowCfg cfg = pick_row_cfg(vec, p.R, max_nl, max_nl, 4, p.mode == kRowLN, three);
  // (rows beyond 64 KB held on one CU also where the row kernels' layouts reach)
  if (int status = 0; cfg.ok && !tune_int("FORCE_STREAM", 0) && p.R / vec > 4096 &&
                      row_onchip_fwd(p, a, vec, st, &status))
    return status;
  if (cfg.ok && !tune_int("FORCE_STREAM", 0)) {
    int grid = cached_grid(p.rows, cfg.tpr);
    // LayerNormalization: a block per row (or per four rows) launches waves
    // faster than they can be started once a row is a few KB - [8192,4096]
    // half: 8192 blocks, 33 us from HBM, 4.0 TB/s.  A few blocks per CU that
    // walk the rows and ask for their next row before they sum the current one:
    // 25 us.  Blocks per CU by measurement (us, block per row -> this):
    // half [12288,4096] 49.0 -> 35.9 with 2, [8192,5120] 42.1 -> 30.8,
    // [16384,3072] 48.9 -> 35.9 with 3 (41.9 with 2), [4096,8192] 29.5 -> 25.7,
    // a wave per row [65536,768] 41.7 -> 36.5 with 3, [16384,1024] 14.8 -> 14.3;
    // float [8192,4096] 49.5 -> 47.3 with 2, [32768,2048] 95.3 -> 89.5 (118.6
    // with 1); not for float rows of a wave or less ([65536,768] 66.6 -> 71.9).
    const bool full = vec == (p.dtype == NBLAHIP_F16 ? 8 : 4);
    if (p.mode == kRowLN && full && cfg.tpr >= 64 && cfg.tpr <= 512 && cfg.nl <= 4 && tune_int("LN_FWD_AHEAD", 1)) {
      const int64_t row_bytes = p.R * (p.dtype == NBLAHIP_F16 ? 2 : 4);
      int per_cu = 0;
      if (cfg.tpr >= 256) per_cu = (p.dtype == NBLAHIP_F16 && row_bytes < 8192) ? 3 : 2;
      else if (p.dtype == NBLAHIP_F16 && cfg.nl >= 2) per_cu = 3;
      per_cu = tune_int("LN_FWD_BLOCKS_PER_CU", per_cu);
      if (per_cu > 0 && grid > 2 * per_cu * device_cus()) {
        RowArgs b = a;
        b.ahead = 1;
        return run_row_fwd_cached(p.dtype, cfg, b, per_cu * device_cus(), st);
      }
    }
    return run_row_fwd_cached(p.dtype, cfg, a, grid, st);
  }
  if (int status = 0; !tune_int("FORCE_STREAM", 0) && row_onchip_fwd(p, a, vec, st, &status))
    return status;
  if (p.dtype == NBLAHIP_F16) {
    return vec == 8   ? stream_fwd_t<__half, 8>(p, a, st)
           : vec == 4 ? stream_fwd_t<__half, 4>(p, a, st)
                      : stream_fwd_t<__half, 1>(p, a, st);
  }
  return vec == 4 ? stream_fwd_t<float, 4>(p, a, st) : stream_fwd_t<float, 1>(p, a, st);
}

// Row chunks of the streaming LayerNormalization column gradients: enough
// (strip, chunk) blocks for 8 per CU, at least 64 rows per chunk.
static int ln_stream_chunks(int64_t rows, int64_t R, int vec = 8) {
  // (the default is the widest strip: the fewest strips, hence the most
  // chunks - the bound the workspace is sized for)
  const int64_t strips = (R + 64 * vec - 1) / (64 * vec);
  const int64_t want = (8 * static_cast<int64_t>(device_cus()) + strips - 1) / strips;
  const int64_t most = std::max<int64_t>(1, rows / 64);
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(std::min(want, most), 65535)));
}

size_t row_bwd_workspace_bytes(int mode, int64_t rows, int64_t R, int64_t planes) {
  if (mode == kRowLN) {
    // Largest persistent grid over the possible thread layouts (one row per
    // block is the 256/1024-thread case).
    const int g = std::max(std::max(ln_bwd_grid(rows, 64), ln_bwd_grid(rows, 256)),
                           std::max(ln_bwd_grid(rows, 512), ln_bwd_grid(rows, 1024)));
    const size_t cached = static_cast<size_t>(g) * 2 * static_cast<size_t>(R) * sizeof(float);
    // row sums, column partials over row chunks, partial sums of split rows
    const size_t split = rows < 2 * static_cast<int64_t>(device_cus())
                             ? static_cast<size_t>(rows) * 64 * 2 * sizeof(float)
                             : 0;
    const size_t stream = align_up(static_cast<size_t>(rows) * 2 * sizeof(float), 256) +
                          align_up(static_cast<size_t>(ln_stream_chunks(rows, R)) * 2 *
                                       static_cast<size_t>(R) * sizeof(float),
                                   256) +
                          split;
    return align_up(std::max(cached, stream), 256);
  }
  // plane pairs, row factors, and the partial pairs of split planes (at most
  // 64 runs each, only taken for fewer than 2 planes per CU)
  const size_t split = planes < 2 * static_cast<int64_t>(device_cus())
                           ? static_cast<size_t>(planes) * 64 * 2 * sizeof(float)
                           : 0;
  return align_up(static_cast<size_t>(planes) * 2 * sizeof(float), 256) +
         align_up(static_cast<size_t>(rows) * 2 * sizeof(float), 256) + align_up(split, 256);
}

// Fold of the LayerNormalization column partials ws[nparts][2][R].  From
// partials of 8 MB on (and rows of whole 16-byte pieces) the kernel that reads
// 256-byte runs; below, the one with 2R/16 blocks, which spreads a small fold
// over more of the chip.
static int launch_ln_param_reduce(const float *ws, int nparts, int R, float *dgamma, float *dbeta,
                                  int accum_g, int accum_b, hipStream_t st) {
  const int64_t bytes = static_cast<int64_t>(nparts) * 2 * R * 4;
  if (R % 4 == 0 && aligned16(ws) &&
      bytes >= static_cast<int64_t>(tune_int("LN_REDUCE_WIDE_MIN_KB", 8192)) * 1024) {
    NBLAHIP_LAUNCH("ln_param_reduce_wide_kernel", ln_param_reduce_wide_kernel, dim3((2 * R + 63) / 64),
                   dim3(1024), 0, st, ws, nparts, R, dgamma, dbeta, accum_g, accum_b);
  } else {
    NBLAHIP_LAUNCH("ln_param_reduce_kernel", ln_param_reduce_kernel, dim3((2 * R + 15) / 16),
                   dim3(1024), 0, st, ws, nparts, R, dgamma, dbeta, accum_g, accum_b);
  }
  return last_launch_status();
}

// LayerNormalization dgamma/dbeta by the streaming kernel: column partials over
// row chunks (kept after the row sums in the workspace), then their fold.
template <typename T, int VEC>
static int stream_ln_colgrad_t(const RowProblem &p, const RowArgs &a, hipStream_t st) {
  float *part = reinterpret_cast<float *>(
      static_cast<char *>(p.ws) + align_up(static_cast<size_t>(p.rows) * 2 * sizeof(float), 256));
  const int Y = ln_stream_chunks(p.rows, p.R, VEC);
  const int rpc = static_cast<int>((p.rows + Y - 1) / Y);
  NBLAHIP_LAUNCH("ln_colgrad_stream_kernel", (ln_colgrad_stream_kernel<T, VEC>),
                 dim3((a.R + 64 * VEC - 1) / (64 * VEC), Y), dim3(256), 0, st,
                 static_cast<const T *>(p.x), static_cast<const T *>(p.dy), p.mean, p.var, a.rows,
                 a.R, rpc, p.eps, part);
  if (int e = last_launch_status()) return e;
  return launch_ln_param_reduce(part, Y, a.R, p.dgamma, p.dbeta, p.accum_g, p.accum_b, st);
}

// vec: the row kernels' vector width for this problem (x and dy aligned, R a
// multiple of it).
static int stream_ln_colgrad(const RowProblem &p, const RowArgs &a, int vec, hipStream_t st) {
  if (p.dtype == NBLAHIP_F16) {
    return vec == 8   ? stream_ln_colgrad_t<__half, 8>(p, a, st)
           : vec == 4 ? stream_ln_colgrad_t<__half, 4>(p, a, st)
                      : stream_ln_colgrad_t<__half, 1>(p, a, st);
  }
  return vec == 4 ? stream_ln_colgrad_t<float, 4>(p, a, st) : stream_ln_colgrad_t<float, 1>(p, a, st);
}

template <typename T, int VEC>
static int stream_bwd_t(const RowProblem &p, const RowArgs &a, hipStream_t st) {
  const T *x = static_cast<const T *>(p.x);
  const T *dy = static_cast<const T *>(p.dy);
  const uint32_t total_vec = static_cast<uint32_t>(p.rows * p.R / VEC);
  const FastDiv nvr(static_cast<uint32_t>(p.R / VEC));
  if (p.mode == kRowLN) {
    float *rs = static_cast<float *>(p.ws);
    if (p.out) {
      const int S = stream_splits(p.rows, p.R / VEC);
      float *split = reinterpret_cast<float *>(
          static_cast<char *>(p.ws) + align_up(static_cast<size_t>(p.rows) * 2 * sizeof(float), 256) +
          align_up(static_cast<size_t>(ln_stream_chunks(p.rows, p.R)) * 2 *
                       static_cast<size_t>(p.R) * sizeof(float),
                   256));
      NBLAHIP_LAUNCH("ln_row_sums_stream_kernel", (ln_row_sums_stream_kernel<T, VEC>),
                     dim3(stream_grid(p.rows), S), dim3(kStreamBlock), 0, st, x, dy, p.gamma,
                     p.mean, a.rows, a.R, S > 1 ? split : rs);
      if (int e = last_launch_status()) return e;
      if (S > 1) {
        NBLAHIP_LAUNCH("pair_split_merge_kernel", pair_split_merge_kernel,
                       dim3(static_cast<unsigned>((p.rows + 63) / 64)), dim3(64), 0, st, split,
                       a.rows, S, rs);
        if (int e = last_launch_status()) return e;
      }
      NBLAHIP_LAUNCH("row_bwd_dx_kernel", (row_bwd_dx_kernel<T, VEC>), dim3(stream_grid((total_vec + 255) / 256)),
                         dim3(256), 0, st, a, rs, nvr, total_vec);
      if (int e = last_launch_status()) return e;
    }
    if (p.dgamma || p.dbeta) return stream_ln_colgrad(p, a, VEC, st);
    return 0;
  }
  const int64_t planes = p.batch * p.channels;
  const int ppr = p.mode == kRowGN ? static_cast<int>(p.channels / p.groups) : 1;
  float *pairs = static_cast<float *>(p.ws);
  float *rs = reinterpret_cast<float *>(static_cast<char *>(p.ws) +
                                        align_up(static_cast<size_t>(planes) * 2 * sizeof(float), 256));
  const int S = stream_splits(planes, p.spatial / VEC);
  float *part = reinterpret_cast<float *>(
      reinterpret_cast<char *>(rs) + align_up(static_cast<size_t>(p.rows) * 2 * sizeof(float), 256));
  NBLAHIP_LAUNCH("plane_sums_stream_kernel", (plane_sums_stream_kernel<T, VEC>),
                 dim3(stream_grid(planes), S), dim3(kStreamBlock), 0, st, x, dy, p.mean,
                 static_cast<int>(planes), static_cast<int>(p.spatial), static_cast<uint32_t>(ppr),
                 S > 1 ? part : pairs);
  if (int e = last_launch_status()) return e;
  if (S > 1) {
    NBLAHIP_LAUNCH("pair_split_merge_kernel", pair_split_merge_kernel,
                   dim3(static_cast<unsigned>((planes + 63) / 64)), dim3(64), 0, st, part,
                   static_cast<int>(planes), S, pairs);
    if (int e = last_launch_status()) return e;
  }
  const uint32_t gmod = (p.mode == kRowGN || p.bc_gamma) ? static_cast<uint32_t>(p.channels) : 0u;
  NBLAHIP_LAUNCH("plane_to_row_factors_kernel", plane_to_row_factors_kernel, dim3(stream_grid(p.rows)), dim3(64), 0, st,
                     pairs, p.gamma, p.var, a.rows, ppr, gmod, p.eps, rs);
  if (int e = last_launch_status()) return e;
  if (p.out) {
    NBLAHIP_LAUNCH("row_bwd_dx_kernel", (row_bwd_dx_kernel<T, VEC>), dim3(stream_grid((total_vec + 255) / 256)),
                       dim3(256), 0, st, a, rs, nvr, total_vec);
    if (int e = last_launch_status()) return e;
  }
  return 0;
}

static int launch_pair_reduce(const RowProblem &p, const float *pairs, hipStream_t st) {
  if (!p.dgamma && !p.dbeta) return 0;
  const int bcg = p.mode == kRowGN ? 1 : p.bc_gamma;
  const int bcb = p.mode == kRowGN ? 1 : p.bc_beta;
  return launch_pair_param_reduce("pair_param_reduce_kernel", pairs, p.batch, p.channels, p.dgamma,
                                  p.dbeta, bcg, bcb, p.accum_g, p.accum_b, st);
}

int launch_row_bwd(const RowProblem &p, hipStream_t st) {
  if (!p.out && !p.dgamma && !p.dbeta) return 0;
  if (int status = 0; !tune_int("FORCE_STREAM", 0) && row_masked_bwd(p, st, &status))
    return status ? status : launch_pair_reduce(p, static_cast<const float *>(p.ws), st);
  const int vec = row_vec(p, true);
  RowArgs a = make_args(p);
  // LayerNormalization also keeps per-column accumulators, gamma and the
  // normalised row in registers.
  const bool ln = p.mode == kRowLN;
  if (!tune_int("FORCE_STREAM", 0) && ln_loose_bwd_wanted(p, vec)) {
    const int full = p.dtype == NBLAHIP_F16 ? 8 : 4;
    // (the kernel for rows at element alignment exists with 1, 2 and 4 vectors per lane)
    const RowCfg loose = pick_ln_bwd_cfg(p.dtype, (p.R + full - 1) / full * full, full, false);
    if (loose.ok && loose.tpr == 64) {
      // (four vectors per lane: 139 - 218 registers, one 512-thread block per CU)
      const int grid = ln_bwd_grid(p.rows, loose.tpr, loose.nl >= 4 ? 1 : 2);
      if (int e = ln_loose_bwd(p, a, loose, grid, st)) return e;
      if (p.dgamma || p.dbeta) {
        if (int e = launch_ln_param_reduce(static_cast<const float *>(p.ws), grid, a.R, p.dgamma,
                                           p.dbeta, p.accum_g, p.accum_b, st))
          return e;
      }
      return 0;
    }
  }
  const int nl_small = ln ? 4 : 8;
  const int nl_1024 = ln ? (p.dtype == NBLAHIP_F16 ? 1 : 2) : 8;
  RowCfg cfg = ln ? pick_ln_bwd_cfg(p.dtype, p.R, vec, true, p.rows)
                  : pick_row_cfg(vec, p.R, nl_small, nl_1024, p.mode == kRowGN ? 256 : 4, false);
  bool gn_map = false;
  if (p.mode == kRowGN) {
    // Fixed map (every wave-wide load of the plain row layout falls inside one
    // channel), with the widest vector or with scalar loads, against the
    // run-time map, by the cost of pick_gn_bwd_cfg; the run-time map pays
    // about 15 % for its address arithmetic (64 KB half groups: 24.5 vs 21.3 us).
    auto cost = [](const RowCfg &c) { return static_cast<int64_t>(c.tpr) * c.nl * (4 + c.vec); };
    RowCfg fixed;
    for (int v : {vec, 1}) {
      const RowCfg c = pick_row_cfg(v, p.R, 8, 8, 256, false);
      if (c.ok && p.spatial % (64 * static_cast<int64_t>(c.vec)) == 0 &&
          (!fixed.ok || cost(c) < cost(fixed)))
        fixed = c;
    }
    RowArgs am = a;
    const RowCfg mapped = pick_gn_bwd_cfg(p, vec, am);
    if (mapped.ok && (!fixed.ok || cost(mapped) * 115 < cost(fixed) * 100)) {
      cfg = mapped;
      a = am;
      gn_map = true;
    } else {
      cfg = fixed;
      if (cfg.ok) a.epc = static_cast<int>(p.spatial / (64 * cfg.vec));
    }
    // The float 1024 x 8 layout (one block per CU, 128 KB of x and as much of
    // dy) lost to the streaming kernels with both in registers (92-105 vs 85 us
    // on 25 088-element groups, 55 vs 56 us on 32 768-element ones); with dy
    // parked in LDS it wins: 80 -> 62 us and 55.5 -> 41 us.
    if (cfg.ok && p.dtype == NBLAHIP_F32 && cfg.vec == 4 && cfg.tpr == 1024 && cfg.nl == 8 &&
        !tune_int("GN_FLOAT_1024X8", 1))
      cfg.ok = false;
  }
  if (!tune_int("FORCE_STREAM", 0)) {
    if (int status = 0; gn_onchip_bwd(p, st, &status))
      return status ? status : launch_pair_reduce(p, static_cast<const float *>(p.ws), st);
  }
  if (!cfg.ok && !tune_int("FORCE_STREAM", 0)) {
    if (int status = 0; in_onchip_bwd(p, st, &status))
      return status ? status : launch_pair_reduce(p, static_cast<const float *>(p.ws), st);
  }
  if (cfg.ok && !tune_int("FORCE_STREAM", 0)) {
    if (p.mode == kRowLN) {
      // A block per row with two or three vectors per thread: the blocks ask
      // for their next row before they work on the current one (cold, us,
      // backward alone / forward + backward in turn: half [8192,5120] 73.7 ->
      // 54.5 / 102.1 -> 95.8, [4096,8192] 55.0 -> 47.0 / 77.2 -> 75.4; float
      // [8192,5120] 102.8 -> 93.8 / 153.1 -> 150.8).  Not with one vector per
      // thread ([16384,3072] half 73.5 -> 76.7) or four (nothing either way), not
      // the other float layouts ([16384,3072] 178.7 -> 183.3 in turn), and not a
      // wave per row: with the next row's vectors the half kernel has one
      // 512-thread block per CU instead of two, which gains 5 % from HBM and
      // loses as much where a step's backward finds x in the Infinity Cache
      // ([65536,768] half 62.5 -> 59.1 alone, 97.6 -> 106.6 in turn; held to 128
      // registers it spills and loses both).  Only where a block has several
      // rows to walk.
      cfg.ahead = ln_bwd_rows_ahead(p.dtype, cfg, vec) && tune_int("LN_BWD_AHEAD", 1);
      int resident = row_bwd_ln_resident_blocks(p.dtype, cfg);
      int grid = ln_bwd_grid(p.rows, cfg.tpr, resident > 0 ? resident : 2);
      const int64_t row_blocks = cfg.tpr <= 64 ? (p.rows + 512 / cfg.tpr - 1) / (512 / cfg.tpr) : p.rows;
      if (cfg.ahead && row_blocks < 2 * static_cast<int64_t>(grid)) {
        cfg.ahead = false;
        resident = row_bwd_ln_resident_blocks(p.dtype, cfg);
        grid = ln_bwd_grid(p.rows, cfg.tpr, resident > 0 ? resident : 2);
      }
      if (int e = run_row_bwd_cached_ln(p.dtype, cfg, a, grid, st)) return e;
      if (p.dgamma || p.dbeta) {
        if (int e = launch_ln_param_reduce(static_cast<const float *>(p.ws), grid, a.R, p.dgamma,
                                           p.dbeta, p.accum_g, p.accum_b, st))
          return e;
      }
      return 0;
    }
    // InstanceNormalization with parameters shared by the batch and enough
    // channels to fill the chip: a block per channel sums over the batch
    // itself, no second kernel.
    // Not with fewer channels than CUs (half the chip idles: [64,128,64,64]
    // float 126 vs 75 us) nor for float planes of 512 vectors and more in
    // batches of 8 and more (10-18 % slower than a row per block plus the
    // batch sum; smaller batches save more on the second launch).
    // Half planes of 512 vectors and more: only with a block for every CU and
    // no second round (us, a block per channel against a row per block plus
    // the batch sum: [16,256,64,64] 20.2 vs 23.2, [32,256,64,64] 37.5 vs 40.6, but
    // [16,320,64,64] 28.5 vs 26.8, [8,1024,64,64] 43.2 vs 40.6), and not beyond
    // 1024 vectors ([16,256,128,128] 84.7 vs 73.5).
    const bool big_float = p.dtype == NBLAHIP_F32 && cfg.tpr * cfg.nl >= 512 && p.batch >= 8;
    const bool big_half = p.dtype == NBLAHIP_F16 && cfg.tpr * cfg.nl >= 512 &&
                          (p.channels > device_cus() || cfg.tpr * cfg.nl > 1024);
    if (p.mode == kRowIN && p.bc_gamma && p.bc_beta && p.batch > 1 &&
        p.channels >= device_cus() && !big_float && !big_half && !(cfg.tpr == 1024 && cfg.nl == 8) &&
        cfg.tpr >= 64 && !tune_int("IN_NO_CHANNEL_BLOCKS", 0)) {
      const int grid = static_cast<int>(std::min<int64_t>(p.channels, 1 << 20));
      return run_row_bwd_cached_inc(p.dtype, cfg, a, grid, st);
    }
    const int grid = cached_grid(p.rows, cfg.tpr);
    const int e = p.mode == kRowIN ? run_row_bwd_cached_in(p.dtype, cfg, a, grid, st)
                  : gn_map         ? run_row_bwd_cached_gnm(p.dtype, cfg, a, grid, st)
                                   : run_row_bwd_cached_gn(p.dtype, cfg, a, grid, st);
    if (e) return e;
    return launch_pair_reduce(p, static_cast<const float *>(p.ws), st);
  }
  if (p.mode == kRowLN && !tune_int("FORCE_STREAM", 0) && tune_int("LN_LONG_ROWS_CACHED", 1)) {
    // Rows too long for the per-column accumulators but not for a block's
    // registers: dx in one pass over x and dy (3 S), the column gradients by
    // the streaming kernel (2 S) - 5 S instead of the 7 S of the all-streaming
    // sequence below.
    // (Not the 1024 x 8 layouts with vectors: 128 KB of row data in one
    // block's registers, 210-256 us against 160-167 us streamed in float,
    // 96 against about 60 us in half.)
    const RowCfg lx = pick_row_cfg(vec, p.R, 8, vec > 1 ? 4 : 8, 256, true);
    if (lx.ok) {
      if (p.out) {
        if (int e = run_row_bwd_cached_lnx(p.dtype, lx, a, cached_grid(p.rows, lx.tpr), st)) return e;
      }
      if (p.dgamma || p.dbeta) return stream_ln_colgrad(p, a, vec, st);
      return 0;
    }
  }
  int e;
  if (p.dtype == NBLAHIP_F16) {
    e = vec == 8   ? stream_bwd_t<__half, 8>(p, a, st)
        : vec == 4 ? stream_bwd_t<__half, 4>(p, a, st)
                   : stream_bwd_t<__half, 1>(p, a, st);
  } else {
    e = vec == 4 ? stream_bwd_t<float, 4>(p, a, st) : stream_bwd_t<float, 1>(p, a, st);
  }
  if (e) return e;
  if (p.mode == kRowLN) return 0;
  return launch_pair_reduce(p, static_cast<const float *>(p.ws), st);
}

// ---------------------------------------------------------------------------
// BatchNormalization through the row kernels: a row is one channel, i.e. its
// N planes of size2 elements.  Taken for the plain training forward and the
// batch-statistics backward when a channel fits the register-cached layouts.
// ---------------------------------------------------------------------------
static bool bn_rows_cfg(const BnProblem &p, bool backward, RowCfg &cfg, RowArgs &a) {
  if (!tune_int("BN_ROWS", 1)) return false;
  if (p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  // channel-last (planes of one element): a row is strided by C, which only a
  // handful of channels keeps inside a cache line (RGB-like inputs); wider
  // channel-last tensors have their own kernels
  if (p.size2 <= 1 && p.C > 8) return false;
  const int64_t R = p.size0 * p.size2;
  if (R < 2 || R > (int64_t{1} << 20)) return false;
  const int64_t bytes = R * p.C * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  const bool tiny = bytes <= (2 << 20); // launches, not bytes, are what costs
  if (p.size2 <= 1 && !tiny) return false;
  int vec = 1;
  const bool al = aligned16(p.x) && (!p.out || aligned16(p.out)) && (!backward || aligned16(p.dy));
  if (al) {
    const int full = p.dtype == NBLAHIP_F16 ? 8 : 4;
    if (p.size2 % full == 0) vec = full;
    else if (p.size2 % 4 == 0) vec = 4;
  }
  // Scalar loads (planes of odd length) pay off for short rows only: beyond,
  // the split path with its tensor-aligned vectors is as fast or faster
  // ([128,2048,7,7] fp16 forward: 34 vs 29 us) - except on tensors so small
  // that its three launches are the cost ([32,64,13,13] fp32: 14 us).
  if (vec == 1 && R > 4096 && !tiny) return false;
  cfg = pick_row_cfg(vec, R, 8, 8, 4, false);
  if (!cfg.ok) return false;
  // a handful of blocks leaves the chip idle: the split reduction spreads
  // such tensors over all CUs - unless the tensor is so small (2 MB) that the
  // three launches of that path are what costs (14 vs 6 us)
  if ((p.C + rows_per_block(cfg.tpr) - 1) / rows_per_block(cfg.tpr) < 32 && !tiny)
    return false;
  a = RowArgs{};
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.rows = static_cast<int>(p.C);
  a.R = static_cast<int>(R);
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / static_cast<double>(R));
  a.one = 1.0f;
  a.percol = 0;
  a.pmod = a.pmod_b = static_cast<uint32_t>(p.C); // parameter index = row
  a.pmul = 1;
  a.pdiv = FastDiv(static_cast<uint32_t>(R));
  a.cpg = 1;
  a.plane = FastDiv(static_cast<uint32_t>(p.size2));
  a.plane_jump = static_cast<uint32_t>((p.C - 1) * p.size2);
  // short planes that share cache lines with their neighbours (bn_onchip.hip
  // has the measurements behind the limit)
  const int64_t plane_bytes = p.size2 * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (plane_bytes % 128 != 0 && plane_bytes <= tune_int("BN_EDGE_STORES_MAX_BYTES", 1024)) {
    a.edge_bytes = static_cast<uint32_t>(plane_bytes);
    const int64_t blocks = cached_grid(p.C, cfg.tpr);
    if (blocks % 8 == 0) a.per_xcd = static_cast<uint32_t>(blocks / 8);
  }
  return true;
}

bool bn_rows_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  RowCfg cfg;
  RowArgs a;
  if (!p.out || !bn_rows_cfg(p, false, cfg, a)) return false;
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  a.decay = p.decay;
  a.unbias = static_cast<float>(N / (N - 1.0));
  *status = run_row_fwd_cached_bn(p.dtype, cfg, a, cached_grid(p.C, cfg.tpr), st);
  return true;
}

bool bn_rows_bwd(const BnProblem &p, hipStream_t st, int *status) {
  RowCfg cfg;
  RowArgs a;
  if (!p.batch_stat || (!p.out && !p.dgamma && !p.dbeta)) return false;
  if (!bn_rows_cfg(p, true, cfg, a)) return false;
  a.mean = const_cast<float *>(p.mean);
  a.var = const_cast<float *>(p.var);
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.accum_dx = p.accum_dx;
  a.dgamma = p.dgamma;
  a.dbeta = p.dbeta;
  a.accum_g = p.accum_g;
  a.accum_b = p.accum_b;
  *status = run_row_bwd_cached_bn(p.dtype, cfg, a, cached_grid(p.C, cfg.tpr), st);
  return true;
}

} // namespace nblahip
