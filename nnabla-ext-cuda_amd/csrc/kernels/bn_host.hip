// Plan selection and launch sequences for BatchNormalization.
#include <algorithm>

#include "bn.cuh"
#include "pair_reduce.cuh"
#include "launch.hpp"

namespace nblahip {

namespace {

struct BnPlan {
  int vec = 1;          // elements per load
  bool channel_last = false;
  // planes layout
  uint32_t nvp = 1;     // vectors per plane
  uint32_t vpc = 1;     // vectors per channel
  uint32_t chunk = 1;   // vectors per split
  // channel-last layout
  uint32_t ncv = 1;     // channel vectors
  uint32_t log2tx = 0;
  uint32_t rps = 1;     // rows per split
  uint32_t ytiles = 1;  // ceil(ncv / TX)
  uint32_t S = 1;       // splits
  int apply_vec = 1;    // vector width of the apply kernels
  bool direct = false;  // planes: one 1024-thread block owns a whole channel (statistics)
  bool direct_bwd = false; // the same for the backward reduction
  // planes whose length is no multiple of the vector width: tensor-aligned
  // vectors, masked at the plane's ends (reductions) or split between the two
  // channels they touch (apply)
  bool masked = false;
  uint32_t size2 = 1;
  uint32_t last_vec = 0;
};

uint32_t ceil_div_u(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

// Upper bound of S over every plan this shape can get (vector width depends on
// pointer alignment, unknown when the workspace is sized).
// Blocks a split reduction aims for.  The planes kernels end with one cheap
// block merge and like many blocks; the channel-last kernels end with an LDS
// fold over 256/TX row groups and like fewer, longer blocks.
uint32_t split_target(bool channel_last, uint64_t tensor_bytes = ~0ull) {
  const uint32_t cus = static_cast<uint32_t>(device_cus());
  if (!channel_last) return cus * tune_int("BN_BLOCKS_PER_CU", 16);
  // Channel-last blocks carry a fixed cost (a partial of C states each, the
  // two-level LDS fold): a block should stream about 96 KB of x, so tensors
  // below ~100 MB get fewer than the 4 blocks per CU of the large ones
  // (25 MB: statistics 13.6 -> 10.8 us, backward reduction 17.4 -> 15.6 us
  // with one block per CU).
  const uint32_t most = static_cast<uint32_t>(tune_int("BN_CL_BLOCKS_PER_CU", 4));
  const uint64_t by_size = tensor_bytes / (96ull << 10) / cus;
  return cus * static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>(most, by_size)));
}

// Vector width of the channel-last kernels: rows of C elements must be a whole
// number of vectors (16 bytes; 8 bytes for fp16 rows of 4k channels).
int cl_vec(int64_t C, int dtype, bool ptr_aligned) {
  if (!ptr_aligned) return 1;
  const int full = dtype == NBLAHIP_F16 ? 8 : 4;
  if (C % full == 0) return full;
  return (dtype == NBLAHIP_F16 && C % 4 == 0) ? 4 : 1;
}

// Grid of a channel-last apply kernel over `slabs` slabs of M rows of ncv
// vectors: column tiles times row blocks, about per_cu blocks per CU in all
// (the kernels load their parameters into registers once per thread, so they
// run as a persistent grid).
struct ClApplyGrid {
  uint32_t x, ntiles;
};
ClApplyGrid cl_apply_grid(uint64_t M, uint32_t ncv, int unroll, int per_cu, uint64_t slabs,
                          uint32_t tile_cols = 256u) {
  ClApplyGrid g;
  const uint32_t cols = std::min(ncv, tile_cols);
  const uint64_t rows_per_step = static_cast<uint64_t>(256u / cols) * unroll;
  g.ntiles = ceil_div_u(ncv, tile_cols);
  const uint64_t need = (M + rows_per_step - 1) / rows_per_step;
  const uint64_t cap =
      per_cu > 0 ? std::max<uint64_t>(1, static_cast<uint64_t>(device_cus()) * per_cu / slabs / g.ntiles)
                 : (1u << 20);
  g.x = g.ntiles * static_cast<uint32_t>(std::max<uint64_t>(1, std::min(need, cap)));
  return g;
}

// Channel vectors per column tile of the forward apply kernel: a power of two
// from 16 (a row segment of 256 bytes) to 256.  A block prepares the parameters
// of its tile's channels before its first load: with 64 vectors (a wave per
// row segment of 1 KiB) [256,7,7,2048] half takes 21 us in inference, with 256
// vectors 26 us (a plain copy 21.5 us).
uint32_t cl_apply_tile_cols(int t) {
  uint32_t c = 16;
  while (c < 256u && static_cast<int>(c) < t) c <<= 1;
  return c;
}

BnPlan make_plan(int64_t size0, int64_t C, int64_t size2, int dtype, bool ptr_aligned) {
  BnPlan pl;
  const int full = dtype == NBLAHIP_F16 ? 8 : 4;
  pl.channel_last = size2 == 1;
  const uint32_t target = split_target(
      pl.channel_last, static_cast<uint64_t>(size0) * C * size2 * (dtype == NBLAHIP_F16 ? 2 : 4));
  if (!pl.channel_last) {
    // Planes of 14x14 = 196 half elements are common: 8-byte accesses there.
    pl.vec = (ptr_aligned && size2 % full == 0)                          ? full
             : (ptr_aligned && dtype == NBLAHIP_F16 && size2 % 4 == 0) ? 4
                                                                        : 1;
    pl.nvp = static_cast<uint32_t>(size2 / pl.vec);
    const uint64_t total = static_cast<uint64_t>(size0) * C * size2;
    if (pl.vec == 1 && ptr_aligned && size2 > full && total % full == 0 &&
        tune_int("BN_MASKED_PLANES", 1)) {
      pl.masked = true;
      pl.vec = full;
      pl.size2 = static_cast<uint32_t>(size2);
      pl.last_vec = static_cast<uint32_t>(total / full - 1);
      pl.nvp = static_cast<uint32_t>((size2 + 2 * full - 2) / full); // most vectors a plane meets
    }
    pl.vpc = static_cast<uint32_t>(size0 * pl.nvp);
    // Enough blocks to fill the chip, but at least one full unrolled step each.
    const uint32_t want = std::max<uint32_t>(1, ceil_div_u(target, static_cast<uint64_t>(C)));
    const uint32_t most = std::max<uint32_t>(1, pl.vpc / (kBnBlock * kBnUnroll));
    uint32_t S = std::min(want, most);
    pl.chunk = ceil_div_u(pl.vpc, S);
    pl.S = ceil_div_u(pl.vpc, pl.chunk);
    // A whole number of channels per CU and enough work per channel: let a
    // 1024-thread block own its channel (no partials, no finalize launch).
    const uint32_t cus = static_cast<uint32_t>(device_cus());
    const int direct = tune_int("BN_DIRECT", 2); // 0 never, 1 always, 2 automatic
    const bool balanced = (static_cast<uint64_t>(C) % cus == 0) || static_cast<uint64_t>(C) >= 8ull * cus;
    // (two steps of the 1024-thread block and more: [32,256,56,56] half, 12 544
    // vectors per channel, 72 vs 81 us forward + backward; smaller channels fit
    // the row kernels' registers and do not come here)
    // The backward reduction takes them from 8192 vectors per channel; the
    // statistics only with one channel per CU below 16 384 (with four rounds of
    // 1024-thread blocks, [256,1024,14,14] half, they lose: 75 vs 64 us forward).
    const bool enough = pl.vpc >= 2u * 1024u * kBnUnroll;
    pl.direct_bwd = direct == 1 || (direct == 2 && balanced && enough);
    pl.direct = direct == 1 || (direct == 2 && balanced && enough &&
                                (pl.vpc >= 4u * 1024u * kBnUnroll || static_cast<uint64_t>(C) <= cus));
  } else {
    pl.vec = cl_vec(C, dtype, ptr_aligned);
    pl.ncv = static_cast<uint32_t>(C / pl.vec);
    uint32_t l2 = 0;
    while ((1u << l2) < pl.ncv && l2 < 6) ++l2; // TX = min(pow2ceil(ncv), 64)
    pl.log2tx = l2;
    const uint32_t TX = 1u << l2;
    const uint32_t TY = kBnBlock >> l2;
    pl.ytiles = ceil_div_u(pl.ncv, TX);
    const uint64_t M = static_cast<uint64_t>(size0);
    // Equal row ranges, a whole number of blocks per CU when the tensor is
    // large enough (an uneven last wave of blocks costs a full block time);
    // the kernels mask the ragged end of a range themselves.
    const uint32_t step = TY * kBnUnroll;
    const uint32_t want = std::max<uint32_t>(1, ceil_div_u(target, pl.ytiles));
    const uint32_t most = std::max<uint32_t>(1, static_cast<uint32_t>(M / step));
    const uint32_t S = std::min(want, most);
    pl.rps = ceil_div_u(M, S);
    pl.S = ceil_div_u(M, pl.rps);
  }
  pl.apply_vec = pl.vec;
  return pl;
}

size_t part_bytes(uint32_t C, uint32_t S) {
  return align_up(static_cast<size_t>(C) * S * 3 * sizeof(float), 256);
}

BnParamSrc param_src(const BnParam *params) {
  BnParamSrc s{};
  s.params = params;
  return s;
}

int apply_grid(uint32_t total_vec, int unroll) {
  const uint64_t blocks = (static_cast<uint64_t>(total_vec) + 256ull * unroll - 1) / (256ull * unroll);
  const int per_cu = tune_int("BN_APPLY_BLOCKS_PER_CU", 0);
  const uint64_t cap = per_cu > 0 ? static_cast<uint64_t>(device_cus()) * per_cu : (1u << 20);
  return static_cast<int>(std::max<uint64_t>(1, std::min<uint64_t>(blocks, cap)));
}

// The widest vector of the element type: only that one has the masked-plane
// kernel variants.
template <typename T, int VEC> constexpr bool kFullVec = VEC == (sizeof(T) == 2 ? 8 : 4);

template <typename T, int VEC, int FUSE>
int fwd_apply_fuse_t(const BnProblem &p, const BnPlan &pl, const BnParamSrc &src, hipStream_t st) {
  const T *x = static_cast<const T *>(p.x);
  const T *z = static_cast<const T *>(p.z);
  T *y = static_cast<T *>(p.out);
  const uint64_t total = static_cast<uint64_t>(p.size0) * p.C * p.size2;
  const uint32_t total_vec = static_cast<uint32_t>(total / VEC);
  if (pl.channel_last) {
    const uint32_t tile_cols = cl_apply_tile_cols(tune_int("BN_CL_FWD_APPLY_TILE", 64));
    const ClApplyGrid g = cl_apply_grid(static_cast<uint64_t>(p.size0), pl.ncv, kBnUnroll,
                                        tune_int("BN_CL_FWD_APPLY_BLOCKS_PER_CU", 4), 1, tile_cols);
    NBLAHIP_LAUNCH(FUSE ? "bn_apply_cl_kernel_fused" : "bn_apply_cl_kernel",
                   (bn_apply_cl_kernel<T, VEC, FUSE>), dim3(g.x), dim3(256), 0, st, x, y, src,
                   pl.ncv, g.ntiles, static_cast<uint32_t>(p.size0), z, 1.0f, tile_cols);
  } else {
    if constexpr (kFullVec<T, VEC>) {
      if (pl.masked) {
        NBLAHIP_LAUNCH(FUSE ? "bn_apply_planes_kernel_fused" : "bn_apply_planes_kernel",
                       (bn_apply_planes_kernel<T, VEC, FUSE, true>),
                       dim3(apply_grid(total_vec, kBnUnroll)), dim3(256), 0, st, x, y, src,
                       FastDiv(pl.size2), FastDiv(static_cast<uint32_t>(p.C)), total_vec, z);
        return last_launch_status();
      }
    }
    NBLAHIP_LAUNCH(FUSE ? "bn_apply_planes_kernel_fused" : "bn_apply_planes_kernel",
                   (bn_apply_planes_kernel<T, VEC, FUSE>), dim3(apply_grid(total_vec, kBnUnroll)),
                   dim3(256), 0, st, x, y, src, FastDiv(pl.nvp),
                   FastDiv(static_cast<uint32_t>(p.C)), total_vec, z);
  }
  return last_launch_status();
}

template <typename T, int VEC>
int fwd_apply_t(const BnProblem &p, const BnPlan &pl, const BnParamSrc &src, hipStream_t st) {
  if (!p.relu) return fwd_apply_fuse_t<T, VEC, 0>(p, pl, src, st);
  return p.z ? fwd_apply_fuse_t<T, VEC, 2>(p, pl, src, st)
             : fwd_apply_fuse_t<T, VEC, 1>(p, pl, src, st);
}

template <typename T, int VEC>
int stats_t(const BnProblem &p, const BnPlan &pl, float *part, const BnFwdFinal &fin,
            hipStream_t st) {
  const T *x = static_cast<const T *>(p.x);
  if (pl.channel_last) {
    NBLAHIP_LAUNCH("bn_stats_cl_kernel", (bn_stats_cl_kernel<T, VEC>), dim3(pl.ytiles, pl.S),
                   dim3(kBnBlock), 0, st, x, static_cast<uint32_t>(p.size0),
                   static_cast<uint32_t>(p.C), pl.ncv, pl.log2tx, pl.rps, 1.0f, part);
  } else if (pl.masked) {
    if constexpr (kFullVec<T, VEC>) {
      if (pl.direct) {
        NBLAHIP_LAUNCH("bn_stats_planes_kernel",
                       (bn_stats_planes_kernel<T, VEC, 1024, true, 4, true>),
                       dim3(static_cast<uint32_t>(p.C), 1), dim3(1024), 0, st, x,
                       static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.vpc, part, fin,
                       pl.size2, pl.last_vec);
      } else {
        NBLAHIP_LAUNCH("bn_stats_planes_kernel",
                       (bn_stats_planes_kernel<T, VEC, kBnBlock, false, kBnUnroll, true>),
                       dim3(static_cast<uint32_t>(p.C), pl.S), dim3(kBnBlock), 0, st, x,
                       static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.chunk, part, fin,
                       pl.size2, pl.last_vec);
      }
    } else {
      return NBLAHIP_EINVAL;
    }
  } else if (pl.direct) {
    NBLAHIP_LAUNCH("bn_stats_planes_kernel", (bn_stats_planes_kernel<T, VEC, 1024, true, 8>),
                   dim3(static_cast<uint32_t>(p.C), 1), dim3(1024), 0, st, x,
                   static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.vpc, part, fin, 0u,
                   0u);
  } else {
    NBLAHIP_LAUNCH("bn_stats_planes_kernel", (bn_stats_planes_kernel<T, VEC, kBnBlock, false, kBnUnroll>),
                   dim3(static_cast<uint32_t>(p.C), pl.S), dim3(kBnBlock), 0, st, x,
                   static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.chunk, part, fin, 0u,
                   0u);
  }
  return last_launch_status();
}

// The reduction also stores the gated dy as dz when that is a plain store: the
// apply step then reads dz in place of (dy, y).
bool gate_in_reduce(const BnProblem &p) { return p.y && p.dz && !p.accum_dz; }

template <typename T, int VEC, bool FUSED>
int bwd_reduce_fuse_t(const BnProblem &p, const BnPlan &pl, float *part2, const BnBwdFinal &fin,
                      hipStream_t st) {
  const T *x = static_cast<const T *>(p.x);
  const T *dy = static_cast<const T *>(p.dy);
  const T *y = static_cast<const T *>(p.y);
  T *dz = gate_in_reduce(p) ? static_cast<T *>(p.dz) : nullptr;
  if (pl.channel_last) {
    NBLAHIP_LAUNCH(FUSED ? "bn_bwd_reduce_cl_kernel_fused" : "bn_bwd_reduce_cl_kernel",
                   (bn_bwd_reduce_cl_kernel<T, VEC, FUSED>), dim3(pl.ytiles, pl.S), dim3(kBnBlock),
                   0, st, x, dy, p.mean, static_cast<uint32_t>(p.size0),
                   static_cast<uint32_t>(p.C), pl.ncv, pl.log2tx, pl.rps, 1.0f, part2, 0u,
                   FastDiv(1), y, dz);
  } else if (pl.masked) {
    if constexpr (kFullVec<T, VEC>) {
      if (pl.direct_bwd) {
        NBLAHIP_LAUNCH(FUSED ? "bn_bwd_reduce_planes_kernel_fused" : "bn_bwd_reduce_planes_kernel",
                       (bn_bwd_reduce_planes_kernel<T, VEC, 1024, true, FUSED, true>),
                       dim3(static_cast<uint32_t>(p.C), 1), dim3(1024), 0, st, x, dy, p.mean,
                       static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.vpc, 1.0f, part2,
                       fin, y, dz, pl.size2, pl.last_vec);
      } else {
        NBLAHIP_LAUNCH(FUSED ? "bn_bwd_reduce_planes_kernel_fused" : "bn_bwd_reduce_planes_kernel",
                       (bn_bwd_reduce_planes_kernel<T, VEC, kBnBlock, false, FUSED, true>),
                       dim3(static_cast<uint32_t>(p.C), pl.S), dim3(kBnBlock), 0, st, x, dy, p.mean,
                       static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.chunk, 1.0f, part2,
                       fin, y, dz, pl.size2, pl.last_vec);
      }
    } else {
      return NBLAHIP_EINVAL;
    }
  } else if (pl.direct_bwd) {
    NBLAHIP_LAUNCH(FUSED ? "bn_bwd_reduce_planes_kernel_fused" : "bn_bwd_reduce_planes_kernel",
                   (bn_bwd_reduce_planes_kernel<T, VEC, 1024, true, FUSED>),
                   dim3(static_cast<uint32_t>(p.C), 1), dim3(1024), 0, st, x, dy, p.mean,
                   static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.vpc, 1.0f, part2, fin,
                   y, dz, 0u, 0u);
  } else {
    NBLAHIP_LAUNCH(FUSED ? "bn_bwd_reduce_planes_kernel_fused" : "bn_bwd_reduce_planes_kernel",
                   (bn_bwd_reduce_planes_kernel<T, VEC, kBnBlock, false, FUSED>),
                   dim3(static_cast<uint32_t>(p.C), pl.S), dim3(kBnBlock), 0, st, x, dy, p.mean,
                   static_cast<uint32_t>(p.C), FastDiv(pl.nvp), pl.vpc, pl.chunk, 1.0f, part2, fin,
                   y, dz, 0u, 0u);
  }
  return last_launch_status();
}

template <typename T, int VEC>
int bwd_reduce_t(const BnProblem &p, const BnPlan &pl, float *part2, const BnBwdFinal &fin,
                 hipStream_t st) {
  return p.y ? bwd_reduce_fuse_t<T, VEC, true>(p, pl, part2, fin, st)
             : bwd_reduce_fuse_t<T, VEC, false>(p, pl, part2, fin, st);
}

template <typename T, int VEC, bool FUSED>
int bwd_apply_fuse_t(const BnProblem &p, const BnPlan &pl, const BnParam *params, hipStream_t st) {
  const T *x = static_cast<const T *>(p.x);
  const T *dy = static_cast<const T *>(p.dy);
  const T *y = static_cast<const T *>(p.y);
  T *dx = static_cast<T *>(p.out);
  T *dz = static_cast<T *>(p.dz);
  const uint64_t total = static_cast<uint64_t>(p.size0) * p.C * p.size2;
  const uint32_t total_vec = static_cast<uint32_t>(total / VEC);
  if (pl.channel_last) {
    const uint32_t tile_cols = cl_apply_tile_cols(tune_int("BN_CL_APPLY_TILE", 64));
    const ClApplyGrid g = cl_apply_grid(static_cast<uint64_t>(p.size0), pl.ncv, 2,
                                        tune_int("BN_CL_APPLY_BLOCKS_PER_CU", 3), 1, tile_cols);
    NBLAHIP_LAUNCH(FUSED ? "bn_bwd_apply_cl_kernel_fused" : "bn_bwd_apply_cl_kernel",
                   (bn_bwd_apply_cl_kernel<T, VEC, FUSED>), dim3(g.x), dim3(256), 0, st, x, dy, dx,
                   params, pl.ncv, g.ntiles, static_cast<uint32_t>(p.size0), p.accum_dx, y, dz,
                   p.accum_dz, tile_cols);
  } else {
    if constexpr (kFullVec<T, VEC>) {
      if (pl.masked) {
        NBLAHIP_LAUNCH(FUSED ? "bn_bwd_apply_planes_kernel_fused" : "bn_bwd_apply_planes_kernel",
                       (bn_bwd_apply_planes_kernel<T, VEC, FUSED, true>),
                       dim3(apply_grid(total_vec, 2)), dim3(256), 0, st, x, dy, dx, params,
                       FastDiv(pl.size2), FastDiv(static_cast<uint32_t>(p.C)), total_vec,
                       p.accum_dx, y, dz, p.accum_dz);
        return last_launch_status();
      }
    }
    NBLAHIP_LAUNCH(FUSED ? "bn_bwd_apply_planes_kernel_fused" : "bn_bwd_apply_planes_kernel",
                   (bn_bwd_apply_planes_kernel<T, VEC, FUSED>), dim3(apply_grid(total_vec, 2)),
                   dim3(256), 0, st, x, dy, dx, params, FastDiv(pl.nvp),
                   FastDiv(static_cast<uint32_t>(p.C)), total_vec, p.accum_dx, y, dz, p.accum_dz);
  }
  return last_launch_status();
}

template <typename T, int VEC>
int bwd_apply_t(const BnProblem &p, const BnPlan &pl, const BnParam *params, hipStream_t st) {
  return p.y ? bwd_apply_fuse_t<T, VEC, true>(p, pl, params, st)
             : bwd_apply_fuse_t<T, VEC, false>(p, pl, params, st);
}

// Run fn<T, VEC>() for the plan's element type and vector width.
#define BN_DISPATCH(CALL, VECV)                                                  \
  do {                                                                           \
    if (p.dtype == NBLAHIP_F16) {                                                \
      if ((VECV) == 8) return CALL(__half, 8);                                   \
      if ((VECV) == 4) return CALL(__half, 4);                                   \
      return CALL(__half, 1);                                                    \
    }                                                                            \
    if ((VECV) == 4) return CALL(float, 4);                                      \
    return CALL(float, 1);                                                       \
  } while (0)

int do_fwd_apply(const BnProblem &p, const BnPlan &pl, const BnParamSrc &src, hipStream_t st) {
#define CALL(T, V) fwd_apply_t<T, V>(p, pl, src, st)
  BN_DISPATCH(CALL, pl.apply_vec);
#undef CALL
}
int do_stats(const BnProblem &p, const BnPlan &pl, float *part, const BnFwdFinal &fin,
             hipStream_t st) {
#define CALL(T, V) stats_t<T, V>(p, pl, part, fin, st)
  BN_DISPATCH(CALL, pl.vec);
#undef CALL
}
int do_bwd_reduce(const BnProblem &p, const BnPlan &pl, float *part2, const BnBwdFinal &fin,
                  hipStream_t st) {
#define CALL(T, V) bwd_reduce_t<T, V>(p, pl, part2, fin, st)
  BN_DISPATCH(CALL, pl.vec);
#undef CALL
}
int do_bwd_apply(const BnProblem &p, const BnPlan &pl, const BnParam *params, hipStream_t st) {
#define CALL(T, V) bwd_apply_t<T, V>(p, pl, params, st)
  BN_DISPATCH(CALL, pl.apply_vec);
#undef CALL
}

} // namespace

size_t bn_workspace_bytes(int64_t size0, int64_t C, int64_t size2, int dtype) {
  // The aligned plan and the scalar plan may pick different S; size for both.
  const BnPlan a = make_plan(size0, C, size2, dtype, true);
  const BnPlan b = make_plan(size0, C, size2, dtype, false);
  const uint32_t S = std::max(a.S, b.S);
  const size_t split_reduction = part_bytes(static_cast<uint32_t>(C), S) +
                                 align_up(static_cast<size_t>(C) * sizeof(BnParam), 256);
  // channel-last tensors through the split kernels: a (sum dy*xh, sum dy) pair
  // per channel and block of the rows
  const size_t split_pairs = size2 == 1 ? static_cast<size_t>(kClSplitMaxBlocks) * C * 2 * sizeof(float) : 0;
  return std::max(split_reduction, split_pairs);
}

int launch_bn_infer(const BnProblem &p, hipStream_t st) {
  const bool al = aligned16(p.x) && aligned16(p.out) && (!p.z || aligned16(p.z));
  const BnPlan pl = make_plan(p.size0, p.C, p.size2, p.dtype, al);
  BnParamSrc src{};
  src.params = nullptr;
  src.rmean = p.mean;
  src.rvar = p.var;
  src.gamma = p.gamma;
  src.beta = p.beta;
  src.eps = p.eps;
  return do_fwd_apply(p, pl, src, st);
}

namespace {
int bn_fwd_train_impl(const BnProblem &p, bool stats_only, hipStream_t st) {
  const bool al = aligned16(p.x) && (stats_only || aligned16(p.out)) && (!p.z || aligned16(p.z));
  const BnPlan pl = make_plan(p.size0, p.C, p.size2, p.dtype, al);
  float *part = static_cast<float *>(p.ws);
  BnParam *params = reinterpret_cast<BnParam *>(static_cast<char *>(p.ws) +
                                                part_bytes(static_cast<uint32_t>(p.C), pl.S));
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  BnFwdFinal fin{};
  fin.inv_N = static_cast<float>(1.0 / N);
  fin.unbias = static_cast<float>(N / (N - 1.0)); // inf when N == 1, as the reference
  fin.decay = p.decay;
  fin.eps = p.eps;
  fin.gamma = p.gamma;
  fin.beta = p.beta;
  fin.batch_mean = p.batch_mean;
  fin.batch_var = p.batch_var;
  fin.rmean = p.rmean;
  fin.rvar = p.rvar;
  fin.params = params;
  if (int e = do_stats(p, pl, part, fin, st)) return e;
  if (!pl.direct) {
    NBLAHIP_LAUNCH("bn_finalize_fwd_kernel", bn_finalize_fwd_kernel,
                   dim3(static_cast<uint32_t>(p.C)), dim3(kBnBlock), 0, st, part, pl.S, fin);
    if (int e = last_launch_status()) return e;
  }
  if (stats_only) return 0;
  return do_fwd_apply(p, pl, param_src(params), st);
}
} // namespace

// Channel-last BatchNormalization as the InstanceNormalization of ONE sample
// whose plane is all the rows: the split kernels (gn_cl_split.hip) take planes
// of up to 65536 positions (64 blocks of 1024), a unit per channel, one pass
// over x per direction.
static bool bn_as_cl_problem(const BnProblem &p, ClProblem &q) {
  if (!tune_int("BN_CL_SPLIT", 1)) return false;
  if (p.size2 != 1 || p.relu || p.z || p.y || p.dz || p.sums_out || p.sums_in) return false;
  if (p.size0 < 2) return false;
  q = ClProblem{};
  q.dtype = p.dtype;
  q.x = p.x;
  q.gamma = p.gamma;
  q.batch = 1;
  q.spatial = p.size0;
  q.channels = p.C;
  q.groups = static_cast<int>(p.C);
  q.eps = p.eps;
  q.ws = p.ws;
  q.ws_bytes = p.ws_bytes;
  q.as_batch_norm = 1;
  return true;
}

bool bn_cl_split_fwd_train(const BnProblem &p, hipStream_t st, int *status) {
  ClProblem q;
  if (!p.out || !bn_as_cl_problem(p, q)) return false;
  q.out = p.out;
  q.beta = p.beta;
  q.mean = p.batch_mean;
  q.var = p.batch_var;
  q.rmean = p.rmean;
  q.rvar = p.rvar;
  q.decay = p.decay;
  const double N = static_cast<double>(p.size0);
  q.unbias = static_cast<float>(N / (N - 1.0));
  return cl_split_fwd(q, aligned16(p.x) && aligned16(p.out), st, status);
}

bool bn_cl_split_bwd(const BnProblem &p, hipStream_t st, int *status) {
  ClProblem q;
  if (!p.batch_stat || !bn_as_cl_problem(p, q)) return false;
  q.dy = p.dy;
  q.out = p.out;
  q.mean = const_cast<float *>(p.mean);
  q.var = const_cast<float *>(p.var);
  q.dmean = p.dmean;
  q.dvar = p.dvar;
  q.dgamma = p.dgamma;
  q.dbeta = p.dbeta;
  q.accum_dx = p.accum_dx;
  float *pairs = nullptr;
  int64_t pair_batches = 0;
  const bool al = aligned16(p.x) && aligned16(p.dy) && (!p.out || aligned16(p.out));
  if (!cl_split_bwd(q, al, &pairs, &pair_batches, st, status)) return false;
  if (*status == 0 && (p.dgamma || p.dbeta))
    *status = launch_pair_param_reduce("pair_param_reduce_cl_kernel", pairs, pair_batches, p.C, p.dgamma,
                                       p.dbeta, 1, 1, p.accum_g, p.accum_b, st);
  return true;
}

int launch_bn_fwd_train(const BnProblem &p, hipStream_t st) {
  int status = 0;
  if (bn_pack_fwd_train(p, st, &status)) return status;
  if (bn_rows_fwd_train(p, st, &status)) return status;
  if (bn_chan_split_fwd_train(p, st, &status)) return status;
  if (bn_onchip_fwd_train(p, st, &status)) return status;
  if (bn_masked_fwd_train(p, st, &status)) return status;
  if (bn_cl_cached_fwd_train(p, st, &status)) return status;
  if (bn_cl_grid_fwd_train(p, st, &status)) return status;
  if (bn_cl_split_fwd_train(p, st, &status)) return status;
  return bn_fwd_train_impl(p, false, st);
}

int launch_bn_local_stats(const BnProblem &p, hipStream_t st) {
  return bn_fwd_train_impl(p, true, st);
}

int launch_bn_merge_stats(const float *stats, int workers, int64_t C, float *batch_mean,
                          float *batch_var, float *rmean, float *rvar, float decay,
                          hipStream_t st) {
  NBLAHIP_LAUNCH("bn_merge_stats_kernel", bn_merge_stats_kernel,
                 dim3(static_cast<uint32_t>((C + 255) / 256)), dim3(256), 0, st, stats,
                 static_cast<uint32_t>(workers), static_cast<uint32_t>(C), batch_mean, batch_var,
                 rmean, rvar, decay);
  return last_launch_status();
}

int launch_bn_bwd(const BnProblem &p, hipStream_t st) {
  if (!p.out && !p.dgamma && !p.dbeta && !p.dz && !p.sums_out) return 0;
  {
    int status = 0;
    if (bn_pack_bwd(p, st, &status)) return status;
    if (bn_rows_bwd(p, st, &status)) return status;
    if (bn_chan_split_bwd(p, st, &status)) return status;
    if (bn_onchip_bwd(p, st, &status)) return status;
    if (bn_masked_bwd(p, st, &status)) return status;
    if (bn_cl_cached_bwd(p, st, &status)) return status;
    if (bn_cl_grid_bwd(p, st, &status)) return status;
    if (bn_cl_split_bwd(p, st, &status)) return status;
  }
  const bool al = aligned16(p.x) && aligned16(p.dy) && (!p.out || aligned16(p.out)) &&
                  (!p.y || aligned16(p.y)) && (!p.dz || aligned16(p.dz));
  const BnPlan pl = make_plan(p.size0, p.C, p.size2, p.dtype, al);
  float *part2 = static_cast<float *>(p.ws);
  BnParam *params = reinterpret_cast<BnParam *>(static_cast<char *>(p.ws) +
                                                part_bytes(static_cast<uint32_t>(p.C), pl.S));
  const bool need_sums = p.dgamma || p.dbeta || p.sums_out || (p.out && p.batch_stat);
  const double N = static_cast<double>(p.size0) * static_cast<double>(p.size2);
  BnBwdFinal fin{};
  fin.inv_N = static_cast<float>(1.0 / N);
  fin.eps = p.eps;
  fin.batch_stat = p.batch_stat;
  fin.gamma = p.gamma;
  fin.mean = p.mean;
  fin.var = p.var;
  fin.dmean_in = p.dmean;
  fin.dvar_in = p.dvar;
  fin.dgamma = need_sums ? p.dgamma : nullptr;
  fin.dbeta = need_sums ? p.dbeta : nullptr;
  fin.accum_g = p.accum_g;
  fin.accum_b = p.accum_b;
  fin.params = params;
  fin.sums = p.sums_out;
  if (need_sums) {
    if (int e = do_bwd_reduce(p, pl, part2, fin, st)) return e;
  }
  // Inference mode, plain BatchNormalization: dx = dy * gamma / std needs neither
  // x nor the sums, so it is the forward's inference apply over dy - 2 S instead
  // of the backward apply's 3 S, and no finalize launch where no parameter
  // gradient is wanted ([32,256,56,56] float, dx alone 57.2 -> 40 us, with
  // dgamma / dbeta 79.5 -> 66).
  const bool infer_dx = !p.batch_stat && p.out && !p.accum_dx && !p.y && !p.dz && !p.z && !p.relu &&
                        tune_int("BN_INFER_BWD_AS_APPLY", 1);
  if (infer_dx) {
    if (need_sums && !pl.direct_bwd) {
      NBLAHIP_LAUNCH("bn_finalize_bwd_kernel", bn_finalize_bwd_kernel,
                     dim3(static_cast<uint32_t>(p.C)), dim3(kBnBlock), 0, st, part2, pl.S, fin);
      if (int e = last_launch_status()) return e;
    }
    BnProblem q = p;
    q.x = p.dy;
    q.dy = nullptr;
    BnParamSrc src{};
    src.params = nullptr;
    src.rmean = nullptr;
    src.rvar = p.var;
    src.gamma = p.gamma;
    src.beta = nullptr;
    src.eps = p.eps;
    return do_fwd_apply(q, pl, src, st);
  }
  if ((p.out || need_sums) && (!need_sums || !pl.direct_bwd)) {
    // Without the reduction (inference-mode dx only) S = 0 leaves the sums at zero.
    NBLAHIP_LAUNCH("bn_finalize_bwd_kernel", bn_finalize_bwd_kernel,
                   dim3(static_cast<uint32_t>(p.C)), dim3(kBnBlock), 0, st, part2,
                   need_sums ? pl.S : 0u, fin);
    if (int e = last_launch_status()) return e;
  }
  if (need_sums && gate_in_reduce(p)) {
    // dz already holds the gated dy: a plain BatchNormalization apply over it.
    if (!p.out) return 0;
    BnProblem q = p;
    q.dy = p.dz;
    q.y = nullptr;
    q.dz = nullptr;
    return do_bwd_apply(q, pl, params, st);
  }
  if (p.out || p.dz) return do_bwd_apply(p, pl, params, st);
  return 0;
}

namespace {
__global__ void __launch_bounds__(256)
sum_rows_kernel(const float *__restrict__ in, int rows, uint32_t n, float *__restrict__ out) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int r = 0; r < rows; ++r) s += in[static_cast<size_t>(r) * n + i];
  out[i] = s;
}
} // namespace

int launch_sum_rows(const float *in, int rows, int64_t n, float *out, hipStream_t st) {
  NBLAHIP_LAUNCH("sum_rows_kernel", sum_rows_kernel, dim3(static_cast<uint32_t>((n + 255) / 256)),
                 dim3(256), 0, st, in, rows, static_cast<uint32_t>(n), out);
  return last_launch_status();
}

int launch_bn_bwd_from_sums(const BnProblem &p, hipStream_t st) {
  if (!p.out) return 0;
  const bool al = aligned16(p.x) && aligned16(p.dy) && aligned16(p.out);
  const BnPlan pl = make_plan(p.size0, p.C, p.size2, p.dtype, al);
  BnParam *params = reinterpret_cast<BnParam *>(static_cast<char *>(p.ws) +
                                                part_bytes(static_cast<uint32_t>(p.C), pl.S));
  BnBwdFinal fin{};
  fin.inv_N = static_cast<float>(1.0 / p.total_count);
  fin.eps = p.eps;
  fin.batch_stat = 1;
  fin.gamma = p.gamma;
  fin.mean = p.mean;
  fin.var = p.var;
  fin.dmean_in = p.dmean;
  fin.dvar_in = p.dvar;
  fin.params = params;
  // The summed pairs are laid out like one split of the partial buffer.
  NBLAHIP_LAUNCH("bn_finalize_bwd_kernel", bn_finalize_bwd_kernel,
                 dim3(static_cast<uint32_t>(p.C)), dim3(kBnBlock), 0, st, p.sums_in, 1u, fin);
  if (int e = last_launch_status()) return e;
  return do_bwd_apply(p, pl, params, st);
}

// ---------------------------------------------------------------------------
// Channel-last Group/InstanceNormalization (N slabs of [S, C]).
// ---------------------------------------------------------------------------
namespace {

BnPlan make_cl_plan(int64_t batch, int64_t spatial, int64_t C, int dtype, bool ptr_aligned) {
  BnPlan pl;
  const int full = dtype == NBLAHIP_F16 ? 8 : 4;
  pl.channel_last = true;
  pl.vec = cl_vec(C, dtype, ptr_aligned);
  pl.ncv = static_cast<uint32_t>(C / pl.vec);
  uint32_t l2 = 0;
  while ((1u << l2) < pl.ncv && l2 < 6) ++l2;
  pl.log2tx = l2;
  const uint32_t TX = 1u << l2;
  const uint32_t TY = kBnBlock >> l2;
  pl.ytiles = ceil_div_u(pl.ncv, TX);
  const uint64_t M = static_cast<uint64_t>(spatial);
  const uint32_t step = TY * kBnUnroll;
  // the batch already multiplies the block count
  const uint64_t per_slab = std::max<uint64_t>(
      1, split_target(true, static_cast<uint64_t>(batch) * spatial * C * (dtype == NBLAHIP_F16 ? 2 : 4)) /
             static_cast<uint64_t>(batch));
  const uint32_t want = std::max<uint32_t>(1, ceil_div_u(per_slab, pl.ytiles));
  const uint32_t most = std::max<uint32_t>(1, static_cast<uint32_t>(M / step));
  const uint32_t S = std::min(want, most);
  pl.rps = ceil_div_u(M, S);
  pl.S = ceil_div_u(M, pl.rps);
  pl.apply_vec = pl.vec;
  return pl;
}

// Groups small enough for one wave each (at most 2 partials per lane: the
// merges of one lane are a serial chain).
bool cl_wave_finalize(uint32_t cpg, uint32_t S) {
  return static_cast<uint64_t>(cpg) * S <= 2u * kWave;
}

struct ClWs {
  float *part;
  BnParam *params;
  float *pairs;
};

size_t cl_part_bytes(int64_t batch, int64_t C, uint32_t S) {
  return align_up(static_cast<size_t>(batch) * C * S * 3 * sizeof(float), 256);
}

ClWs cl_carve(const ClProblem &p, const BnPlan &pl) {
  ClWs w;
  char *base = static_cast<char *>(p.ws);
  w.part = reinterpret_cast<float *>(base);
  base += cl_part_bytes(p.batch, p.channels, pl.S);
  w.params = reinterpret_cast<BnParam *>(base);
  base += align_up(static_cast<size_t>(p.batch) * p.channels * sizeof(BnParam), 256);
  w.pairs = reinterpret_cast<float *>(base);
  return w;
}

template <typename T, int VEC>
int cl_stats_t(const ClProblem &p, const BnPlan &pl, float *part, hipStream_t st) {
  NBLAHIP_LAUNCH("bn_stats_cl_kernel", (bn_stats_cl_kernel<T, VEC>),
                 dim3(pl.ytiles, pl.S, static_cast<uint32_t>(p.batch)), dim3(kBnBlock), 0, st,
                 static_cast<const T *>(p.x), static_cast<uint32_t>(p.spatial),
                 static_cast<uint32_t>(p.channels), pl.ncv, pl.log2tx, pl.rps, 1.0f, part);
  return last_launch_status();
}

template <typename T, int VEC>
int cl_apply_t(const ClProblem &p, const BnPlan &pl, const BnParam *params, hipStream_t st) {
  const ClApplyGrid g = cl_apply_grid(static_cast<uint64_t>(p.spatial), pl.ncv, kBnUnroll,
                                      tune_int("BN_CL_APPLY_BLOCKS_PER_CU", 3),
                                      static_cast<uint64_t>(p.batch));
  NBLAHIP_LAUNCH("bn_apply_cl_kernel", (bn_apply_cl_kernel<T, VEC>),
                 dim3(g.x, static_cast<uint32_t>(p.batch)), dim3(256), 0, st,
                 static_cast<const T *>(p.x), static_cast<T *>(p.out), param_src(params), pl.ncv,
                 g.ntiles, static_cast<uint32_t>(p.spatial), static_cast<const T *>(nullptr), 1.0f,
                 256u);
  return last_launch_status();
}

template <typename T, int VEC>
int cl_bwd_reduce_t(const ClProblem &p, const BnPlan &pl, float *part2, hipStream_t st) {
  const uint32_t cpg = static_cast<uint32_t>(p.channels / p.groups);
  NBLAHIP_LAUNCH("bn_bwd_reduce_cl_kernel", (bn_bwd_reduce_cl_kernel<T, VEC>),
                 dim3(pl.ytiles, pl.S, static_cast<uint32_t>(p.batch)), dim3(kBnBlock), 0, st,
                 static_cast<const T *>(p.x), static_cast<const T *>(p.dy), p.mean,
                 static_cast<uint32_t>(p.spatial), static_cast<uint32_t>(p.channels), pl.ncv,
                 pl.log2tx, pl.rps, 1.0f, part2, static_cast<uint32_t>(p.groups), FastDiv(cpg),
                 static_cast<const T *>(nullptr), static_cast<T *>(nullptr));
  return last_launch_status();
}

template <typename T, int VEC>
int cl_bwd_apply_t(const ClProblem &p, const BnPlan &pl, const BnParam *params, hipStream_t st) {
  const uint32_t tile_cols = cl_apply_tile_cols(tune_int("BN_CL_APPLY_TILE", 64));
  const ClApplyGrid g = cl_apply_grid(static_cast<uint64_t>(p.spatial), pl.ncv, 2,
                                      tune_int("BN_CL_APPLY_BLOCKS_PER_CU", 3),
                                      static_cast<uint64_t>(p.batch), tile_cols);
  NBLAHIP_LAUNCH("bn_bwd_apply_cl_kernel", (bn_bwd_apply_cl_kernel<T, VEC>),
                 dim3(g.x, static_cast<uint32_t>(p.batch)), dim3(256), 0, st,
                 static_cast<const T *>(p.x), static_cast<const T *>(p.dy), static_cast<T *>(p.out),
                 params, pl.ncv, g.ntiles, static_cast<uint32_t>(p.spatial), p.accum_dx,
                 static_cast<const T *>(nullptr), static_cast<T *>(nullptr), 0, tile_cols);
  return last_launch_status();
}

} // namespace

size_t cl_workspace_bytes(int64_t batch, int64_t spatial, int64_t channels, int dtype) {
  const BnPlan a = make_cl_plan(batch, spatial, channels, dtype, true);
  const BnPlan b = make_cl_plan(batch, spatial, channels, dtype, false);
  const size_t split_reduction = cl_part_bytes(batch, channels, std::max(a.S, b.S)) +
                                 align_up(static_cast<size_t>(batch) * channels * sizeof(BnParam), 256) +
                                 align_up(static_cast<size_t>(batch) * channels * 2 * sizeof(float), 256);
  // the split kernels (gn_cl_split.hip): a pair per channel and block of a plane
  const size_t split_pairs = static_cast<size_t>(batch) * kClSplitMaxBlocks * channels * 2 * sizeof(float);
  return std::max(split_reduction, split_pairs);
}

// Groups whose channel count keeps them from the split kernels: whether the
// tile kernels (blocks of whole rows, a block per CU) are tried before the
// cached ones (a block per group, 16-byte pieces of the rows).  The cached
// kernels win on small groups and on tensors of a few MB (one short launch
// without an exchange); vectors per group from which the tile kernels are ahead,
// on 8-60 MB tensors from HBM: half forward 2048 ([16,36,36,400] G=25 15.9 against
// 14.8 us, [16,48,48,200] 18.2 / 14.3, [16,64,64,200] 28.0 / 17.6; below,
// [16,32,32,400] 13.4 / 13.7, [16,28,28,200] 8.8 / 12.6), half backward 768
// ([16,28,28,200] 17.6 / 16.7, [16,32,32,200] 20.0 / 16.9, [16,40,40,200] 25.0 / 18.3;
// below, [16,24,24,200] 15.7 / 16.5), float forward 768 ([32,28,28,100] G=25
// 12.7 / 11.4, [32,40,40,100] 22.4 / 14.2; below, [32,20,20,100] 8.2 / 10.1), float
// backward 512 ([32,24,24,100] 18.0 / 15.2, [32,32,32,72] G=9 18.9 / 16.1; below,
// [32,16,16,72] 10.2 / 12.3).
static bool cl_tile_first(const ClProblem &p, bool backward) {
  if (p.groups == p.channels) return false;
  const bool half = p.dtype == NBLAHIP_F16;
  const int64_t vec = half ? 8 : 4;
  const int64_t cpg = p.channels / p.groups;
  if (cpg % vec != 0) return false;
  if (p.channels % (8 * vec) == 0) return false; // whole 128-byte lines: not measured here
  if (p.batch * p.spatial * p.channels * (half ? 2 : 4) <= (4 << 20)) return false;
  const int64_t nv = p.spatial * (cpg / vec);
  const int64_t from = half ? (backward ? tune_int("GN_CL_TILE_FIRST_BWD", 768)
                                        : tune_int("GN_CL_TILE_FIRST_FWD", 2048))
                            : (backward ? tune_int("GN_CL_TILE_FIRST_BWD_F32", 512)
                                        : tune_int("GN_CL_TILE_FIRST_FWD_F32", 768));
  return nv > from;
}

int launch_cl_fwd(const ClProblem &p, hipStream_t st) {
  const bool al = aligned16(p.x) && aligned16(p.out);
  {
    int status = 0;
    if (cl_split_fwd(p, al, st, &status)) return status;
    if (cl_tile_first(p, false) && cl_tile_fwd(p, al, st, &status)) return status;
    if (gn_cl_cached_fwd(p, al, st, &status)) return status;
    if (cl_tile_fwd(p, al, st, &status)) return status;
  }
  const BnPlan pl = make_cl_plan(p.batch, p.spatial, p.channels, p.dtype, al);
  const ClWs w = cl_carve(p, pl);
  const uint32_t cpg = static_cast<uint32_t>(p.channels / p.groups);
#define CALL(T, V) cl_stats_t<T, V>(p, pl, w.part, st)
  const int e1 = [&]() -> int { BN_DISPATCH(CALL, pl.vec); }();
#undef CALL
  if (e1) return e1;
  const float inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * cpg));
  const uint32_t NG = static_cast<uint32_t>(p.batch * p.groups);
  if (cl_wave_finalize(cpg, pl.S)) {
    NBLAHIP_LAUNCH("gn_cl_finalize_fwd_kernel", gn_cl_finalize_fwd_kernel<true>,
                   dim3(ceil_div_u(NG, kBnBlock / kWave)), dim3(kBnBlock), 0, st, w.part, pl.S,
                   static_cast<uint32_t>(p.channels), cpg, NG, inv_R, p.eps, p.gamma, p.beta,
                   p.bc_gamma ? 1u : 0u, p.bc_beta ? 1u : 0u, p.mean, p.var, w.params);
  } else {
    NBLAHIP_LAUNCH("gn_cl_finalize_fwd_kernel", gn_cl_finalize_fwd_kernel<false>, dim3(NG),
                   dim3(kBnBlock), 0, st, w.part, pl.S, static_cast<uint32_t>(p.channels), cpg, NG,
                   inv_R, p.eps, p.gamma, p.beta, p.bc_gamma ? 1u : 0u, p.bc_beta ? 1u : 0u,
                   p.mean, p.var, w.params);
  }
  if (int e = last_launch_status()) return e;
#define CALL(T, V) cl_apply_t<T, V>(p, pl, w.params, st)
  BN_DISPATCH(CALL, pl.apply_vec);
#undef CALL
}

int launch_cl_bwd(const ClProblem &p, hipStream_t st) {
  if (!p.out && !p.dgamma && !p.dbeta) return 0;
  const bool al = aligned16(p.x) && aligned16(p.dy) && (!p.out || aligned16(p.out));
  const BnPlan pl = make_cl_plan(p.batch, p.spatial, p.channels, p.dtype, al);
  const ClWs w = cl_carve(p, pl);
  {
    int status = 0;
    float *pairs = nullptr;
    int64_t pair_batches = 0;
    if (cl_split_bwd(p, al, &pairs, &pair_batches, st, &status)) {
      if (status) return status;
      if (p.dgamma || p.dbeta)
        return launch_pair_param_reduce("pair_param_reduce_cl_kernel", pairs, pair_batches,
                                        p.channels, p.dgamma, p.dbeta, 1, 1, p.accum_g, p.accum_b, st);
      return 0;
    }
    auto after_tile = [&]() -> int {
      if (status) return status;
      if (p.dgamma || p.dbeta)
        return launch_pair_param_reduce("pair_param_reduce_cl_kernel", pairs, pair_batches,
                                        p.channels, p.dgamma, p.dbeta, 1, 1, p.accum_g, p.accum_b, st);
      return 0;
    };
    if (cl_tile_first(p, true) && cl_tile_bwd(p, al, &pairs, &pair_batches, st, &status))
      return after_tile();
    if (gn_cl_cached_bwd(p, al, w.pairs, st, &status)) {
      if (status) return status;
      if (p.dgamma || p.dbeta)
        return launch_pair_param_reduce("pair_param_reduce_cl_kernel", w.pairs, p.batch, p.channels,
                                        p.dgamma, p.dbeta, p.bc_gamma, p.bc_beta, p.accum_g,
                                        p.accum_b, st);
      return 0;
    }
    if (cl_tile_bwd(p, al, &pairs, &pair_batches, st, &status)) return after_tile();
  }
  const uint32_t cpg = static_cast<uint32_t>(p.channels / p.groups);
#define CALL(T, V) cl_bwd_reduce_t<T, V>(p, pl, w.part, st)
  const int e1 = [&]() -> int { BN_DISPATCH(CALL, pl.vec); }();
#undef CALL
  if (e1) return e1;
  const float inv_R = static_cast<float>(1.0 / (static_cast<double>(p.spatial) * cpg));
  const uint32_t NG = static_cast<uint32_t>(p.batch * p.groups);
  uint32_t sp = 1; // lanes sharing the splits of one channel: power of two, at most a wave
  while (sp < pl.S && sp < kWave) sp <<= 1;
  if (cl_wave_finalize(cpg, pl.S)) {
    NBLAHIP_LAUNCH("gn_cl_finalize_bwd_kernel", gn_cl_finalize_bwd_kernel<true>,
                   dim3(ceil_div_u(NG, kBnBlock / kWave)), dim3(kBnBlock), 0, st, w.part, pl.S, sp,
                   static_cast<uint32_t>(p.channels), cpg, NG, inv_R, p.eps, p.gamma,
                   p.bc_gamma ? 1u : 0u, p.mean, p.var, p.dmean, p.dvar, w.pairs, w.params);
  } else {
    NBLAHIP_LAUNCH("gn_cl_finalize_bwd_kernel", gn_cl_finalize_bwd_kernel<false>, dim3(NG),
                   dim3(kBnBlock), 0, st, w.part, pl.S, sp, static_cast<uint32_t>(p.channels), cpg,
                   NG, inv_R, p.eps, p.gamma, p.bc_gamma ? 1u : 0u, p.mean, p.var, p.dmean, p.dvar,
                   w.pairs, w.params);
  }
  if (int e = last_launch_status()) return e;
  if (p.out) {
#define CALL(T, V) cl_bwd_apply_t<T, V>(p, pl, w.params, st)
    const int e2 = [&]() -> int { BN_DISPATCH(CALL, pl.apply_vec); }();
#undef CALL
    if (e2) return e2;
  }
  if (p.dgamma || p.dbeta) {
    if (int e = launch_pair_param_reduce("pair_param_reduce_cl_kernel", w.pairs, p.batch, p.channels,
                                         p.dgamma, p.dbeta, p.bc_gamma, p.bc_beta, p.accum_g,
                                         p.accum_b, st))
      return e;
  }
  return 0;
}

} // namespace nblahip
