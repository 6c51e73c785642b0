// Instantiations and launcher of the register-cached channel-last
// GroupNormalization kernels.
#include <algorithm>

#include "gn_cl_rows.cuh"

namespace nblahip {

// gn_cl_rows_fused.hip
int run_in_fwd_fused(int dtype, int tpr, int nl, const GnClArgs &a, unsigned grid, int fuse,
                     hipStream_t st);
int run_in_bwd_fused(int dtype, int tpr, int nl, const GnClArgs &a, unsigned grid, hipStream_t st);

namespace {

struct GnClCfg {
  bool ok = false;
  int vec = 1, tpr = 256, nl = 1;
};

// Whether the blocks of gpl neighbouring units go to one XCD (GN_CL_XCD_MAP:
// 0 never, 2 only where gpl divides the units of a sample).  Where it does not
// divide them the sets of gpl units lie askew to the cache lines, and a line
// still has two XCDs fetching it instead of up to eight: [15,64,64,200] half
// instances forward 47.8 us without the map.
bool xcd_map_for(int64_t units_per_sample, int64_t gpl) {
  const int mode = tune_int("GN_CL_XCD_MAP", 1);
  return mode == 1 || (mode == 2 && units_per_sample % gpl == 0);
}

// The cached kernels apply when a group is at least one vector of channels
// wide (cpg = VEC * cvg, cvg in {1, 2, 4, 8}), fits 8 loads per thread of a
// block, and is big enough to be worth a block; parameters shared by the batch.
GnClCfg pick_cfg(const ClProblem &p, bool aligned, bool backward, GnClArgs &a) {
  GnClCfg c;
  if (!aligned || !tune_int("GN_CL_CACHED", 1)) return c;
  if (!p.bc_gamma || !p.bc_beta) return c;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  const int64_t cpg = p.channels / p.groups;
  if (cpg % vec != 0) return c;
  const int64_t cvg = cpg / vec;
  if (cvg != 1 && cvg != 2 && cvg != 4 && cvg != 8) return c;
  const int64_t nv = p.spatial * cvg;
  if (nv < 32) return c;
  // Backward, beyond 2048 vectors per group the three-kernel path is as fast
  // or faster (64 KB half groups: 41.9 vs 42.4 us; 50 KB ones: 56.1 vs 52.6 us),
  // the strided 16-byte accesses of two tensors being the limit; below it the
  // single pass wins clearly (28x28 planes: 24 vs 39 us).
  if (backward && nv > 2048) return c;
  // small groups: one wave per group (no LDS, no barrier), at most 4 loads
  for (int tpr : {64, 256, 512, 1024}) {
    for (int nl : {1, 2, 4, 8}) {
      if (static_cast<int64_t>(tpr) * nl < nv) continue;
      if (tpr == 64 && nl > 4) continue;
      // the float 1024 x 8 layout (128 KB of x and dy in one block's registers)
      // is left to the three-kernel path
      if (p.dtype == NBLAHIP_F32 && tpr == 1024 && nl == 8) continue;
      c.ok = true;
      c.vec = vec;
      c.tpr = tpr;
      c.nl = nl;
      break;
    }
    if (c.ok) break;
  }
  if (!c.ok) return c;
  a.P = static_cast<int>(p.spatial);
  a.C = static_cast<int>(p.channels);
  a.G = p.groups;
  a.cpg = static_cast<int>(cpg);
  a.units = static_cast<int>(p.batch * p.groups);
  a.cvg = FastDiv(static_cast<uint32_t>(cvg));
  const int64_t line = 128 / (p.dtype == NBLAHIP_F16 ? 2 : 4); // elements per 128-byte line
  const int64_t gpl = line / cpg;
  a.gpl = (gpl >= 2 && xcd_map_for(p.groups, gpl)) ? static_cast<int>(gpl) : 1;
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * cpg));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  return c;
}

// InstanceNormalization: a block per (sample, channel vector); P positions of
// one vector each.
GnClCfg pick_in_cfg(const ClProblem &p, bool aligned, bool backward, GnClArgs &a,
                    int64_t min_positions = -1) {
  GnClCfg c;
  if (!aligned || !tune_int("IN_CL_CACHED", 1)) return c;
  if (!p.bc_gamma || !p.bc_beta) return c;
  const int vec = p.dtype == NBLAHIP_F16 ? 8 : 4;
  if (p.channels % vec != 0) return c;
  const int64_t nv = p.spatial;
  if (nv < (min_positions >= 0 ? min_positions : tune_int("IN_CL_MIN", 32))) return c;
  // Beyond 2048 positions the three-kernel path is as fast or faster in float
  // and in the backward pass (64x64 planes, half: backward 49 vs 44 us; 56x56
  // float: 62 / 130 vs 57 / 92 us).
  if ((backward || p.dtype == NBLAHIP_F32) && nv > 2048) return c;
  // InstanceNormalization proper, tensors beyond a few MB (below, the single
  // launch wins), planes from which the three-kernel path is ahead from HBM,
  // this against it: half forward 2048 positions ([28,48,48,200] 28.8 vs 25.7 us,
  // [15,64,64,200] 29.2 vs 24.4; below, [40,40,40,200] 26.2 vs 28.0), float forward
  // 1024 ([32,36,36,100] 20.6 vs 18.4, [32,40,40,100] 24.1 vs 20.1; below,
  // [32,32,32,100] 16.4 vs 16.8), float backward 640 ([32,28,28,100] 19.9 vs 18.7,
  // [32,32,32,72] 19.6 vs 18.5; below, [32,24,24,100] 16.4 vs 17.6).
  if (min_positions < 0 &&
      p.batch * p.spatial * p.channels * (p.dtype == NBLAHIP_F16 ? 2 : 4) > (4 << 20)) {
    const int64_t most = p.dtype == NBLAHIP_F16 ? tune_int("IN_CL_MAX", 2048)
                         : backward             ? tune_int("IN_CL_MAX_F32_BWD", 640)
                                                : tune_int("IN_CL_MAX_F32_FWD", 1024);
    if (nv > most) return c;
  }
  for (int tpr : {64, 256, 512, 1024}) {
    for (int nl : {1, 2, 4, 8}) {
      if (static_cast<int64_t>(tpr) * nl < nv) continue;
      if (tpr == 64 && nl > 4) continue; // one wave per unit: at most 4 loads
      if (p.dtype == NBLAHIP_F32 && tpr == 1024 && nl == 8) continue;
      c.ok = true;
      c.vec = vec;
      c.tpr = tpr;
      c.nl = nl;
      break;
    }
    if (c.ok) break;
  }
  if (!c.ok) return c;
  a.P = static_cast<int>(p.spatial);
  a.C = static_cast<int>(p.channels);
  a.G = static_cast<int>(p.channels / vec);
  a.cpg = vec;
  a.units = static_cast<int>(p.batch * a.G);
  a.cvg = FastDiv(1);
  const int gpl = 128 / (vec * (p.dtype == NBLAHIP_F16 ? 2 : 4)); // vectors per 128-byte line
  a.gpl = xcd_map_for(a.G, gpl) ? gpl : 1;
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / static_cast<double>(p.spatial));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  return c;
}

unsigned grid_of(const GnClArgs &a) {
  if (a.gpl <= 1) return static_cast<unsigned>(a.units);
  const unsigned sets = static_cast<unsigned>((a.units + a.gpl - 1) / a.gpl);
  return (sets + kXcds - 1) / kXcds * kXcds * static_cast<unsigned>(a.gpl);
}

#define GN_CL_CASES_TPR(CASE, T, VEC, TPR) \
  CASE(T, VEC, 1, TPR) CASE(T, VEC, 2, TPR) CASE(T, VEC, 4, TPR) CASE(T, VEC, 8, TPR)
#define GN_CL_CASES(CASE, T, VEC) \
  GN_CL_CASES_TPR(CASE, T, VEC, 256) GN_CL_CASES_TPR(CASE, T, VEC, 512) GN_CL_CASES_TPR(CASE, T, VEC, 1024)
// ... and one wave per unit (small planes or groups).
#define IN_CL_CASES(CASE, T, VEC) GN_CL_CASES_TPR(CASE, T, VEC, 64) GN_CL_CASES(CASE, T, VEC)
// The backwards take groups / planes of up to 2048 vectors (pick_cfg,
// pick_in_cfg), which the wave and the 256-thread layouts hold: the larger
// blocks are never picked.
#define CL_CASES_BWD(CASE, T, VEC) GN_CL_CASES_TPR(CASE, T, VEC, 64) GN_CL_CASES_TPR(CASE, T, VEC, 256)

#define FWD_CASE(T, VEC, NL, TPR)                                                              \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                        \
    NBLAHIP_LAUNCH("gn_cl_row_fwd_kernel", (gn_cl_row_fwd_kernel<T, VEC, NL, TPR>),            \
                   dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    return last_launch_status();                                                               \
  }
#define BWD_CASE(T, VEC, NL, TPR)                                                              \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                        \
    NBLAHIP_LAUNCH("gn_cl_row_bwd_kernel", (gn_cl_row_bwd_kernel<T, VEC, NL, TPR>),            \
                   dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    return last_launch_status();                                                               \
  }

#define IN_FWD_CASE(T, VEC, NL, TPR)                                                           \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                        \
    NBLAHIP_LAUNCH("in_cl_row_fwd_kernel", (in_cl_row_fwd_kernel<T, VEC, NL, TPR>),            \
                   dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    return last_launch_status();                                                               \
  }
#define IN_BWD_CASE(T, VEC, NL, TPR)                                                           \
  if (c.nl == (NL) && c.tpr == (TPR)) {                                                        \
    NBLAHIP_LAUNCH("in_cl_row_bwd_kernel", (in_cl_row_bwd_kernel<T, VEC, NL, TPR>),            \
                   dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    return last_launch_status();                                                               \
  }

int run_in_fwd(int dtype, const GnClCfg &c, const GnClArgs &a, hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    IN_CL_CASES(IN_FWD_CASE, __half, 8)
  } else {
    IN_CL_CASES(IN_FWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

int run_in_bwd(int dtype, const GnClCfg &c, const GnClArgs &a, hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    CL_CASES_BWD(IN_BWD_CASE, __half, 8)
  } else {
    CL_CASES_BWD(IN_BWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

int run_fwd(int dtype, const GnClCfg &c, const GnClArgs &a, hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    IN_CL_CASES(FWD_CASE, __half, 8)
  } else {
    IN_CL_CASES(FWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

int run_bwd(int dtype, const GnClCfg &c, const GnClArgs &a, hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    CL_CASES_BWD(BWD_CASE, __half, 8)
  } else {
    CL_CASES_BWD(BWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

} // namespace

namespace {

// Wide forward (half data, planes of 1024 positions and more): the widest
// chunk - 4 or 2 neighbouring groups / channel vectors per block, 64 or 32
// bytes per position - that still leaves a block for every CU and fits a
// block's registers.
template <int W>
int run_wide(bool instance, int tpr, int nl, const GnClArgs &a, hipStream_t st) {
#define WIDE_CASE(NL, TPR)                                                                       \
  if (nl == (NL) && tpr == (TPR)) {                                                              \
    if (instance) {                                                                              \
      NBLAHIP_LAUNCH("in_cl_wide_fwd_kernel",                                                    \
                     (in_cl_wide_fwd_kernel<__half, 8, NL, TPR, W, (NL) * (TPR) == 8192>),       \
                     dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    } else {                                                                                     \
      NBLAHIP_LAUNCH("gn_cl_wide_fwd_kernel", (gn_cl_wide_fwd_kernel<__half, 8, NL, TPR, W>),    \
                     dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    }                                                                                            \
    return last_launch_status();                                                                 \
  }
  WIDE_CASE(4, 512)
  WIDE_CASE(8, 512)
  WIDE_CASE(4, 1024)
  WIDE_CASE(8, 1024)
#undef WIDE_CASE
  // 16 vectors per thread: GroupNormalization only (the instance kernel keeps
  // 8 statistics per thread beside its vectors and would spill)
  if (nl == 16 && tpr == 1024 && !instance) {
    NBLAHIP_LAUNCH("gn_cl_wide_fwd_kernel", (gn_cl_wide_fwd_kernel<__half, 8, 16, 1024, W>),
                   dim3(grid_of(a)), dim3(1024), 0, st, a);
    return last_launch_status();
  }
  return NBLAHIP_EINVAL;
}

bool wide_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status) {
  if (!aligned || p.dtype != NBLAHIP_F16 || !tune_int("GN_CL_WIDE", 1)) return false;
  if (!p.bc_gamma || !p.bc_beta || p.spatial < 1024) return false;
  constexpr int vec = 8;
  const bool instance = p.groups == p.channels;
  const int64_t cpg = instance ? vec : p.channels / p.groups; // channels of one unit of the chunk
  if (cpg % vec != 0 || p.channels % vec != 0) return false;
  const int64_t cvg = cpg / vec;                               // vectors per unit
  // Only 16-byte pieces gain: from 32-byte pieces on it is a wash or a loss
  // ([64,32,32,512] in 32 groups 28.3 -> 29.9 us, [64,32,32,256] in 8 groups 13.5 -> 15.9 us).
  if (cvg != 1) return false;
  const int64_t per_sample = instance ? p.channels / vec : p.groups; // units per sample
  for (int w : {4, 2}) {
    if (per_sample % w != 0 || cvg * w > 8) continue;
    const int64_t blocks = p.batch * (per_sample / w);
    const int64_t nv = p.spatial * cvg * w; // vectors a block holds
    // A block for every CU, except where four groups of a long plane (16
    // vectors per thread, GroupNormalization only) leave one for every other
    // CU: 64-byte pieces from half the CUs beat 32-byte pieces from all of them
    // ([16,64,64,256] G=32: 19.0 -> 17.8 us).
    const bool long_tile = w == 4 && !instance && nv > 8192;
    if (blocks * 100 < static_cast<int64_t>(device_cus()) * tune_int("GN_CL_WIDE_MIN_PCT", long_tile ? 50 : 100))
      continue;
    for (int tpr : {512, 1024}) {
      for (int nl : {4, 8, 16}) {
        if (nl == 16 && (tpr != 1024 || instance)) continue;
        if (static_cast<int64_t>(tpr) * nl < nv) continue;
        GnClArgs a{};
        a.x = p.x;
        a.out = p.out;
        a.gamma = p.gamma;
        a.beta = p.beta;
        a.mean = p.mean;
        a.var = p.var;
        a.P = static_cast<int>(p.spatial);
        a.C = static_cast<int>(p.channels);
        a.G = static_cast<int>(per_sample / w);
        a.groups = static_cast<int>(per_sample);
        a.cpg = static_cast<int>(cpg);
        a.units = static_cast<int>(blocks);
        a.cvg = FastDiv(static_cast<uint32_t>(cvg));
        a.chunk = FastDiv(static_cast<uint32_t>(cvg * w));
        const int64_t gpl = 128 / (cpg * w * 2); // blocks sharing a 128-byte line
        a.gpl = (gpl >= 2 && xcd_map_for(a.G, gpl)) ? static_cast<int>(gpl) : 1;
        a.eps = p.eps;
        a.inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * (instance ? 1 : cpg)));
        a.one = 1.0f;
        *status = w == 4 ? run_wide<4>(instance, tpr, nl, a, st) : run_wide<2>(instance, tpr, nl, a, st);
        return true;
      }
    }
  }
  return false;
}

} // namespace

bool gn_cl_cached_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status) {
  if (wide_fwd(p, aligned, st, status)) return true;
  GnClArgs a{};
  const bool instance = p.groups == p.channels;
  const GnClCfg c = instance ? pick_in_cfg(p, aligned, false, a) : pick_cfg(p, aligned, false, a);
  if (!c.ok) return false;
  a.x = p.x;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.mean = p.mean;
  a.var = p.var;
  *status = instance ? run_in_fwd(p.dtype, c, a, st) : run_fwd(p.dtype, c, a, st);
  return true;
}

namespace {

template <int W>
int run_wide_bwd(bool instance, int tpr, int nl, const GnClArgs &a, hipStream_t st) {
#define WIDE_CASE(NL, TPR)                                                                       \
  if (nl == (NL) && tpr == (TPR)) {                                                              \
    if (instance) {                                                                              \
      NBLAHIP_LAUNCH("cl_wide_bwd_kernel", (cl_wide_bwd_kernel<NL, TPR, W, true>),               \
                     dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    } else {                                                                                     \
      NBLAHIP_LAUNCH("cl_wide_bwd_kernel", (cl_wide_bwd_kernel<NL, TPR, W, false>),              \
                     dim3(grid_of(a)), dim3(TPR), 0, st, a);                                     \
    }                                                                                            \
    return last_launch_status();                                                                 \
  }
  WIDE_CASE(4, 512)
  WIDE_CASE(8, 512)
  WIDE_CASE(4, 1024)
  WIDE_CASE(8, 1024)
#undef WIDE_CASE
  return NBLAHIP_EINVAL;
}

// Same shapes as the wide forward (half data, 8 channels per group or
// instances, planes of 1024 positions and more, a block for every CU left).
bool wide_bwd(const ClProblem &p, bool aligned, float *pairs, hipStream_t st, int *status) {
  if (!aligned || p.dtype != NBLAHIP_F16 || !tune_int("GN_CL_WIDE_BWD", 1)) return false;
  if (!p.bc_gamma || !p.bc_beta || p.spatial < 1024) return false;
  constexpr int vec = 8;
  const bool instance = p.groups == p.channels;
  if (p.channels % vec != 0 || (!instance && p.channels / p.groups != vec)) return false;
  const int64_t per_sample = instance ? p.channels / vec : p.groups;
  for (int w : {4, 2}) {
    if (per_sample % w != 0) continue;
    const int64_t blocks = p.batch * (per_sample / w);
    if (blocks < device_cus()) continue;
    const int64_t nv = p.spatial * w;
    for (int tpr : {512, 1024}) {
      for (int nl : {4, 8}) {
        if (static_cast<int64_t>(tpr) * nl < nv) continue;
        GnClArgs a{};
        a.x = p.x;
        a.dy = p.dy;
        a.out = p.out;
        a.gamma = p.gamma;
        a.mean = p.mean;
        a.var = p.var;
        a.dmean = p.dmean;
        a.dvar = p.dvar;
        a.pairs = pairs;
        a.P = static_cast<int>(p.spatial);
        a.C = static_cast<int>(p.channels);
        a.G = static_cast<int>(per_sample / w);
        a.groups = static_cast<int>(per_sample);
        a.cpg = vec;
        a.units = static_cast<int>(blocks);
        const int64_t gpl = 128 / (vec * w * 2); // blocks sharing a 128-byte line
        a.gpl = (gpl >= 2 && xcd_map_for(a.G, gpl)) ? static_cast<int>(gpl) : 1;
        a.eps = p.eps;
        a.inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * (instance ? 1 : vec)));
        a.one = 1.0f;
        a.accum_dx = p.accum_dx;
        *status = w == 4 ? run_wide_bwd<4>(instance, tpr, nl, a, st)
                         : run_wide_bwd<2>(instance, tpr, nl, a, st);
        return true;
      }
    }
  }
  return false;
}

} // namespace

bool gn_cl_cached_bwd(const ClProblem &p, bool aligned, float *pairs, hipStream_t st,
                      int *status) {
  if (wide_bwd(p, aligned, pairs, st, status)) return true;
  GnClArgs a{};
  const bool instance = p.groups == p.channels;
  const GnClCfg c = instance ? pick_in_cfg(p, aligned, true, a) : pick_cfg(p, aligned, true, a);
  if (!c.ok) return false;
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.pairs = pairs;
  *status = instance ? run_in_bwd(p.dtype, c, a, st) : run_bwd(p.dtype, c, a, st);
  return true;
}

// ---------------------------------------------------------------------------
// Channel-last BatchNormalization [M, C] with few rows: the instance kernels
// with one "sample" of M positions; a block per channel vector keeps its
// column of the tensor in registers (one launch, 2 S / 3 S).
// ---------------------------------------------------------------------------
static bool bn_cl_cfg(const BnProblem &p, bool backward, GnClCfg &c, GnClArgs &a) {
  if (!tune_int("BN_CL_CACHED", 1)) return false;
  if (p.size2 != 1 || p.sums_out || p.sums_in) return false;
  const bool al = aligned16(p.x) && (!p.out || aligned16(p.out)) && (!backward || aligned16(p.dy)) &&
                  (!p.z || aligned16(p.z)) && (!p.y || aligned16(p.y)) && (!p.dz || aligned16(p.dz));
  ClProblem q;
  q.dtype = p.dtype;
  q.batch = 1;
  q.spatial = p.size0;
  q.channels = p.C;
  q.groups = static_cast<int>(p.C);
  q.eps = p.eps;
  q.accum_dx = p.accum_dx;
  // The single pass wins up to 1024 rows and 4 MiB, and on anything up to
  // 1 MiB; beyond, the split kernels (forward + backward us from HBM, this
  // against them: half [1024,1024] 15.9 vs 17.9, [1024,4096] 26.5 vs 22.6,
  // [1568,2048] 24.6 vs 20.7, [4096,1024] 31.8 vs 24.3; float [1568,4096] 66.1 vs
  // 35.7, [2048,2048] 44.5 vs 27.8; a block per channel vector walks the rows
  // alone).
  c = pick_in_cfg(q, al, backward, a, 2); // also the few rows of a fully connected layer's batch
  if (!c.ok) return false;
  // a handful of blocks: the split reduction fills the chip (tensors of up to
  // 2 MB excepted: there its three launches cost more than idle CUs)
  const int64_t bytes = p.size0 * p.C * (p.dtype == NBLAHIP_F16 ? 2 : 4);
  if (a.units < 32 && bytes > (2 << 20)) return false;
  // (FusedBatchNormalization has no split kernels to fall to: up to 2048 rows,
  // the forward up to 4096 with at least 64 blocks, against its three-kernel path)
  if (p.z || p.relu || p.y || p.dz) return !(p.size0 > 2048 && (p.size0 > 4096 || a.units < 64));
  if (bytes > (1 << 20)) {
    if (p.size0 > tune_int("BN_CL_CACHED_MAX_ROWS", 1024) ||
        bytes >= static_cast<int64_t>(tune_int("BN_CL_CACHED_MAX_KB", 4096)) * 1024)
      return false;
  } else if (p.size0 > 2048) {
    return false;
  }
  return true;
}

bool bn_cl_cached_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  GnClCfg c;
  GnClArgs a{};
  if (!p.out || !bn_cl_cfg(p, false, c, a)) return false;
  const double N = static_cast<double>(p.size0);
  a.x = p.x;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.mean = p.batch_mean;
  a.var = p.batch_var;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  a.decay = p.decay;
  a.unbias = static_cast<float>(N / (N - 1.0));
  a.z = p.z;
  *status = !p.relu ? run_in_fwd(p.dtype, c, a, st)
                    : run_in_fwd_fused(p.dtype, c.tpr, c.nl, a, grid_of(a), p.z ? 2 : 1, st);
  return true;
}

bool bn_cl_cached_bwd(const BnProblem &p, hipStream_t st, int *status) {
  GnClCfg c;
  GnClArgs a{};
  if (!p.batch_stat || (!p.out && !p.dgamma && !p.dbeta && !p.dz)) return false;
  if (!bn_cl_cfg(p, true, c, a)) return false;
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.mean = const_cast<float *>(p.mean);
  a.var = const_cast<float *>(p.var);
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.direct_params = 1;
  a.dgamma = p.dgamma;
  a.dbeta = p.dbeta;
  a.accum_g = p.accum_g;
  a.accum_b = p.accum_b;
  a.y = p.y;
  a.dz = p.dz;
  a.accum_dz = p.accum_dz;
  *status = !p.y ? run_in_bwd(p.dtype, c, a, st)
                 : run_in_bwd_fused(p.dtype, c.tpr, c.nl, a, grid_of(a), st);
  return true;
}

} // namespace nblahip
