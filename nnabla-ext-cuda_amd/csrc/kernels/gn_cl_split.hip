// Host side of the split channel-last Group/InstanceNormalization kernels
// (gn_cl_split.cuh): eligibility, the block shape, the exchange array and the
// per-call epoch.
#include <algorithm>

#include "gn_cl_split.cuh"

namespace nblahip {

namespace {

struct SplitPlan {
  bool ok = false;
  bool instance = false;
  int vec = 8, tpr = 512, nl = 8;
  int tiles = 0, split = 0, pb = 0, cpg = 1, cvg_shift = 0, units = 0; // units per tile
  size_t words = 0;
};

SplitPlan plan_split(const ClProblem &p, bool aligned, bool backward) {
  SplitPlan s;
  if (!aligned || !tune_int("GN_CL_SPLIT", 1)) return s;
  if (!p.bc_gamma || !p.bc_beta) return s;
  // Instances exchange 64 channels x 2 words per block and partner: the polls
  // cost what the whole lines save (C4 stored NHWC forward 27 vs 22 us), so
  // they stay with the kernels of gn_cl_rows.cuh unless asked for.
  if (p.groups == p.channels && !tune_int("GN_CL_SPLIT_INSTANCES", 0)) return s;
  const int esz = p.dtype == NBLAHIP_F16 ? 2 : 4;
  s.vec = 16 / esz;
  const int64_t tile_ch = static_cast<int64_t>(kSplitTV) * s.vec; // channels of a 128-byte line
  if (p.channels % tile_ch != 0) return s;
  s.instance = p.groups == p.channels;
  s.cpg = static_cast<int>(p.channels / p.groups);
  if (!s.instance) {
    if (s.cpg % s.vec != 0) return s;
    const int cvg = s.cpg / s.vec;
    if (cvg != 1 && cvg != 2 && cvg != 4 && cvg != 8) return s;
    while ((1 << s.cvg_shift) < cvg) ++s.cvg_shift;
  }
  s.units = s.instance ? static_cast<int>(tile_ch) : kSplitTV >> s.cvg_shift;
  s.tiles = static_cast<int>(p.channels / tile_ch);
  // Block shape: positions per block PB = NL * TPR / 8.  256 threads x 8
  // vectors (32 KB of half data, four blocks to a CU) is the fastest shape in
  // both directions over a sweep of shapes (C4 stored NHWC backward 25.5 us
  // against 31.5 with 512 x 8, whose half instantiation spills); the forward of
  // long planes and float data gain a little from 512 x 8 (15.6 vs 16.4 us,
  // float backward 40.0 vs 43.0 us).  Planes beyond 16 blocks of the largest
  // shape are left to the other kernels.
  static const int shapes[][2] = {{256, 4}, {256, 8}, {512, 8}, {1024, 8}, {512, 4}, {1024, 4}};
  const int ftpr = tune_int("GN_CL_SPLIT_TPR", 0), fnl = tune_int("GN_CL_SPLIT_NL", 0);
  const bool forced = ftpr && fnl;
  const bool large_first = p.spatial >= 4096 && (!backward || p.dtype == NBLAHIP_F32);
  for (int pass = 0; pass < 2 && !s.ok; ++pass) {
    for (int i = 0; i < (forced ? 6 : 4); ++i) {
      const int *sh = shapes[i];
      if (forced && (sh[0] != ftpr || sh[1] != fnl)) continue;
      const int64_t pb = static_cast<int64_t>(sh[0]) * sh[1] / kSplitTV;
      const int64_t split = (p.spatial + pb - 1) / pb;
      if (split > kSplitMax) continue;
      if (!forced) {
        if (pass == 0 && large_first && sh[0] != 512) continue; // first choice for these
        if (i == 0 && p.spatial > pb) continue;                 // 256 x 4 only for planes it holds whole
      }
      s.tpr = sh[0];
      s.nl = sh[1];
      s.pb = static_cast<int>(pb);
      s.split = static_cast<int>(split);
      s.ok = true;
      break;
    }
    if (!large_first || forced) break;
  }
  if (!s.ok) return s;
  const int64_t blocks = p.batch * s.tiles * static_cast<int64_t>(s.split);
  s.words = static_cast<size_t>(blocks) * 2 * s.units;
  if (blocks > (1ll << 30) || s.words > xchg_capacity()) s.ok = false;
  if (backward &&
      static_cast<size_t>(p.batch) * s.split * p.channels * 2 * sizeof(float) > p.ws_bytes)
    s.ok = false;
  return s;
}

ClSplitArgs make_args(const ClProblem &p, const SplitPlan &s) {
  ClSplitArgs a{};
  a.x = p.x;
  a.dy = p.dy;
  a.out = p.out;
  a.gamma = p.gamma;
  a.beta = p.beta;
  a.mean = p.mean;
  a.var = p.var;
  a.dmean = p.dmean;
  a.dvar = p.dvar;
  a.spin = tune_int("XCHG_SPIN", 64);
  a.P = static_cast<int>(p.spatial);
  a.C = static_cast<int>(p.channels);
  a.tiles = s.tiles;
  a.split = s.split;
  a.PB = s.pb;
  a.cpg = s.instance ? 1 : s.cpg;
  a.cvg_shift = s.cvg_shift;
  a.eps = p.eps;
  a.inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * (s.instance ? 1 : s.cpg)));
  a.one = 1.0f;
  a.accum_dx = p.accum_dx;
  return a;
}

template <typename T, int VEC, bool INSTANCE>
int run(bool backward, const SplitPlan &s, const ClSplitArgs &a, unsigned grid, hipStream_t st) {
#define SPLIT_CASE(TPR, NL)                                                                      \
  if (s.tpr == (TPR) && s.nl == (NL)) {                                                          \
    if (backward) {                                                                              \
      NBLAHIP_LAUNCH("cl_split_bwd_kernel", (cl_split_bwd_kernel<T, VEC, NL, TPR, INSTANCE>),    \
                     dim3(grid), dim3(TPR), 0, st, a);                                           \
    } else {                                                                                     \
      NBLAHIP_LAUNCH("cl_split_fwd_kernel", (cl_split_fwd_kernel<T, VEC, NL, TPR, INSTANCE>),    \
                     dim3(grid), dim3(TPR), 0, st, a);                                           \
    }                                                                                            \
    return last_launch_status();                                                                 \
  }
  SPLIT_CASE(256, 4)
  SPLIT_CASE(256, 8)
  SPLIT_CASE(512, 4)
  SPLIT_CASE(512, 8)
  SPLIT_CASE(1024, 4)
  SPLIT_CASE(1024, 8)
#undef SPLIT_CASE
  return NBLAHIP_EINVAL;
}

int dispatch(const ClProblem &p, const SplitPlan &s, bool backward, const ClSplitArgs &a,
             hipStream_t st) {
  const unsigned grid = static_cast<unsigned>(p.batch * s.tiles * s.split);
  if (p.dtype == NBLAHIP_F16) {
    return s.instance ? run<__half, 8, true>(backward, s, a, grid, st)
                      : run<__half, 8, false>(backward, s, a, grid, st);
  }
  return s.instance ? run<float, 4, true>(backward, s, a, grid, st)
                    : run<float, 4, false>(backward, s, a, grid, st);
}

} // namespace

bool cl_split_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status) {
  const SplitPlan s = plan_split(p, aligned, false);
  if (!s.ok) return false;
  ClSplitArgs a = make_args(p, s);
  if (!xchg_acquire(s.words, st, &a.xchg, &a.epoch, status)) return *status != 0;
  *status = dispatch(p, s, false, a, st);
  return true;
}

bool cl_split_bwd(const ClProblem &p, bool aligned, float **pairs, int64_t *pair_batches,
                  hipStream_t st, int *status) {
  const SplitPlan s = plan_split(p, aligned, true);
  if (!s.ok) return false;
  ClSplitArgs a = make_args(p, s);
  if (!xchg_acquire(s.words, st, &a.xchg, &a.epoch, status)) return *status != 0;
  a.pairs = static_cast<float *>(p.ws); // [batch * split][C][2], summed over its first axis afterwards
  *pairs = a.pairs;
  *pair_batches = p.batch * s.split;
  *status = dispatch(p, s, true, a, st);
  return true;
}

} // namespace nblahip
