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
  bool partners_adjacent = false;
  int64_t lds_bytes = 0;
};

SplitPlan plan_split(const ClProblem &p, bool aligned, bool backward) {
  SplitPlan s;
  if (!aligned) return s;
  if (!p.as_batch_norm) { // (BatchNormalization has its own switch)
    if (!tune_int("GN_CL_SPLIT", 1)) return s;
    if (p.groups == p.channels && !tune_int("GN_CL_SPLIT_INSTANCES", 1)) return s;
  }
  if (!p.bc_gamma || !p.bc_beta) return s;
  const int esz = p.dtype == NBLAHIP_F16 ? 2 : 4;
  // A block whose partner's word does not arrive reads the partner's part of x
  // (and dy) again, which the partner may already be overwriting in place.
  const uint64_t tensor_bytes = static_cast<uint64_t>(p.batch * p.spatial * p.channels) * esz;
  if (ranges_overlap(p.out, p.x, tensor_bytes) || (backward && ranges_overlap(p.out, p.dy, tensor_bytes)))
    return s;
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
  // Block shape: positions per block PB = NL * TPR / 8 (128, 256, 512 or 1024);
  // planes beyond 16 blocks of the largest shape are left to the other kernels
  // (BatchNormalization's single plane of all rows: beyond 64 blocks).
  // First choice, from sweeps of the shapes (cold, forward / backward us):
  //  forward: several blocks to a CU, so that one block's exchange and stores
  //    run while the next one's loads arrive - groups 256 x 8 (float and planes
  //    from 4096 positions: 512 x 8; [16,64,64,256] half 13.7 vs 14.3), instances
  //    512 x 8 ([16,64,64,256] 15.2 against 17.1 with 1024 x 8), 256 x 8 where
  //    512 x 8 leaves CUs without a block ([4,32,32,1024] 7.9 vs 8.8);
  //  backward: 1024 x 8, one block per CU (dy waits in 128 KB of LDS), for
  //    instances and for groups whose plane one such block holds whole, where
  //    that gives every CU a block and the plane's last block is not mostly
  //    empty ([16,64,64,256] instances 22.8 vs 25.0; [32,28,28,512] groups
  //    17.5 vs 20.2; but [32,56,56,128] instances, 3136 = 3 x 1024 + 64
  //    positions, 22.1 vs 20.4); else 512 x 8 where that still gives two blocks
  //    per CU (instances: one), else 256 x 8 ([4,32,32,1024] 11.1 vs 11.6);
  //  any plane that one block of a smaller shape holds whole takes that shape.
  static const int shapes[][2] = {{256, 4}, {256, 8}, {512, 8}, {1024, 8}, {512, 4}, {1024, 4}};
  const int ftpr = tune_int("GN_CL_SPLIT_TPR", 0), fnl = tune_int("GN_CL_SPLIT_NL", 0);
  const bool forced = ftpr && fnl;
  auto take = [&](int i) {
    const int64_t pb = static_cast<int64_t>(shapes[i][0]) * shapes[i][1] / kSplitTV;
    const int64_t split = (p.spatial + pb - 1) / pb;
    // (more than 16 blocks per plane only for BatchNormalization's single plane
    // of all rows, and only in the largest blocks: the partials a block collects
    // grow with the number of its partners)
    if (split > (p.as_batch_norm && i == 3 ? kSplitMax : 16)) return false;
    s.lds_bytes = 16 * 1024; // forward: folds and partials, far from the limit
    if (backward) {
      // LDS of cl_split_bwd_kernel: dy parked, the folds, and the blocks'
      // partials (sized by the launch) - together at most the CU's 160 KB
      const int64_t ch = tile_ch, umax = s.instance ? ch : kSplitTV;
      const int64_t fixed = static_cast<int64_t>(shapes[i][0]) * shapes[i][1] * 16 +
                            (shapes[i][0] / 64) * 2 * ch * 4 + 2 * ch * 4 + umax * 2 * 4 + ch * 4 +
                            kSplitMax * 4 + 256;
      const int64_t partials = (split > 16 ? split : 16) * 2 * umax * 4;
      if (fixed + partials > 160 * 1024) return false;
      s.lds_bytes = fixed + partials;
    }
    s.tpr = shapes[i][0];
    s.nl = shapes[i][1];
    s.pb = static_cast<int>(pb);
    s.split = static_cast<int>(split);
    s.ok = true;
    return true;
  };
  if (forced) {
    for (int i = 0; i < 6 && !s.ok; ++i)
      if (shapes[i][0] == ftpr && shapes[i][1] == fnl) take(i);
  } else {
    const int64_t cus = device_cus();
    auto blocks_of = [&](int i) {
      const int64_t pb = static_cast<int64_t>(shapes[i][0]) * shapes[i][1] / kSplitTV;
      return p.batch * s.tiles * ((p.spatial + pb - 1) / pb);
    };
    auto well_filled = [&](int i) { // the plane's blocks hold at least 90 % of their positions
      const int64_t pb = static_cast<int64_t>(shapes[i][0]) * shapes[i][1] / kSplitTV;
      return p.spatial * 10 >= ((p.spatial + pb - 1) / pb) * pb * 9;
    };
    int first = 1; // 256 x 8
    if (p.spatial <= 128) {
      first = 0;
    } else if (p.spatial <= 256) {
      first = 1;
    } else if (backward && blocks_of(3) >= cus && well_filled(3) && (s.instance || p.spatial <= 1024)) {
      first = 3;
    } else if (s.instance) {
      first = blocks_of(2) >= cus ? 2 : 1;
    } else if (backward) {
      if (blocks_of(2) >= 2 * cus) first = 2;
    } else if (p.spatial >= 4096 || (p.dtype == NBLAHIP_F32 && p.spatial >= 2048)) {
      first = 2;
    }
    for (int i = first; i < 4 && !s.ok; ++i) take(i);
  }
  if (!s.ok) return s;
  const int64_t blocks = p.batch * s.tiles * static_cast<int64_t>(s.split);
  // More blocks than the chip holds at once (a CU takes 1024 threads of these
  // kernels, and what its LDS allows): a block's partners must be its
  // neighbours in the grid, or they are not running yet when it polls for
  // their parts.
  const int64_t per_cu = std::max<int64_t>(1, std::min<int64_t>(1024 / s.tpr, 160 * 1024 / s.lds_bytes));
  s.partners_adjacent = blocks > device_cus() * per_cu;
  // With more than 16 partners a grid of several rounds stalls on the planes
  // that straddle two rounds ([256,14,14,1024] half forward, 49 blocks per
  // column tile, 784 in all: 80 us against 62 us of the split reduction).
  if (s.split > 16 && s.partners_adjacent) s.ok = false;
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
  a.partners_adjacent = s.partners_adjacent ? 1 : 0;
  a.rmean = p.rmean;
  a.rvar = p.rvar;
  a.decay = p.decay;
  a.unbias = p.unbias;
  return a;
}

template <typename T, int VEC, bool INSTANCE>
int run(bool backward, const SplitPlan &s, const ClSplitArgs &a, unsigned grid, hipStream_t st) {
  // the blocks' partials of every unit of a tile, in LDS
  const size_t part_bytes = static_cast<size_t>(s.split) * 2 * s.units * sizeof(float);
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
  if constexpr (INSTANCE) {
    if (s.split > 16) { // (planned only in the largest block shape)
      if (s.tpr != 1024 || s.nl != 8) return NBLAHIP_EINVAL;
      if (backward) {
        NBLAHIP_LAUNCH("cl_split_bwd_kernel", (cl_split_bwd_kernel<T, VEC, 8, 1024, true, true>),
                       dim3(grid), dim3(1024), part_bytes, st, a);
      } else {
        NBLAHIP_LAUNCH("cl_split_fwd_kernel", (cl_split_fwd_kernel<T, VEC, 8, 1024, true, true>),
                       dim3(grid), dim3(1024), part_bytes, st, a);
      }
      return last_launch_status();
    }
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
