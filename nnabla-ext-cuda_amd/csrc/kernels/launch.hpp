// Host-side launch layer shared by the translation units of the kernel
// library: problem descriptions, plan selection and the internal launch
// functions the C-ABI entry points call.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include "../../../include/nblahip.h"

namespace nblahip {

// kRowINc: InstanceNormalization backward with a block per channel that walks
// the batch itself, so dgamma/dbeta need no second kernel.
// kRowGNm: GroupNormalization backward with the run-time thread map (planes
// that are no multiple of a wave-wide load); kRowGN is the fixed map.
// kRowBN: BatchNormalization of tensors whose channel (all its planes) fits a
// block's registers: a row is the strided set of planes of one channel.
// kRowLNx: LayerNormalization backward of rows too long for the per-column
// accumulators of kRowLN: dx only (gamma read per row), the column gradients
// come from the streaming kernel.
enum RowMode {
  kRowLN = 0,
  kRowIN = 1,
  kRowGN = 2,
  kRowINc = 3,
  kRowGNm = 4,
  kRowBN = 5,
  kRowLNx = 6
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// True when the byte ranges [a, a + bytes) and [b, b + bytes) share a byte
// (null pointers overlap nothing).  The kernels whose blocks may recompute a
// partner's partial sums from global memory read tensors that the partner is
// already overwriting when the output shares memory with an input, so their
// plans turn such calls down and the kernels without an exchange take them.
inline bool ranges_overlap(const void *a, const void *b, uint64_t bytes) {
  if (!a || !b || bytes == 0) return false;
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return pa < pb ? pb - pa < bytes : pa - pb < bytes;
}

// Number of compute units of the current device (cached per device).
int device_cus();

// Integer plan knob (name without the prefix "NBLAHIP_"): the value set through
// nblahip_tune_set, else the environment's (read once), else `fallback`.
int tune_int(const char *name, int fallback);

// One row-normalization problem (LayerNormalization rows,
// InstanceNormalization planes or GroupNormalization groups).
struct RowProblem {
  int dtype = 0;
  int mode = 0; // RowMode
  const void *x = nullptr;
  const void *dy = nullptr;
  void *out = nullptr; // y or dx
  const float *gamma = nullptr;
  const float *beta = nullptr;
  float *mean = nullptr;
  float *var = nullptr;
  const float *dmean = nullptr;
  const float *dvar = nullptr;
  float *dgamma = nullptr;
  float *dbeta = nullptr;
  int accum_dx = 0, accum_g = 0, accum_b = 0;
  int64_t rows = 0; // statistics rows
  int64_t R = 0;    // elements per statistics row
  // GN / IN geometry: x is [batch, channels, spatial]
  int64_t batch = 1, channels = 1, spatial = 1;
  int groups = 1;
  int bc_gamma = 1, bc_beta = 1;
  float eps = 0.f;
  void *ws = nullptr;
  size_t ws_bytes = 0;
};

// Register-cached configuration: TPR threads per row, NL loads of vec elements each.
// InstanceNormalization backward with a plane's x held on one CU (bn_onchip.hip);
// false: not taken.  Leaves the per-plane (dgamma, dbeta) parts in p.ws.
bool in_onchip_bwd(const RowProblem &p, hipStream_t st, int *status);
// GroupNormalization backward with a group of 128 - 336 KB held on one CU
// (gn_onchip_bwd.hip); false: not taken.  Leaves the per-(sample, channel)
// (dgamma, dbeta) parts in p.ws.
bool gn_onchip_bwd(const RowProblem &p, hipStream_t st, int *status);

struct RowCfg {
  bool ok = false;
  int vec = 1, tpr = 64, nl = 1;
  bool ahead = false; // LayerNormalization backward: the kernel that asks for its next row ahead
};

// vec: elements per load (alignment and divisibility already checked by the
// caller).  max_nl / max_nl_1024 bound the loads per thread below / at 1024
// threads; min_tpr is 256 for the GroupNormalization backward and 4 where
// several rows may share a wave; percol: LayerNormalization parameter layout.
RowCfg pick_row_cfg(int vec, int64_t R, int max_nl, int max_nl_1024, int min_tpr, bool percol,
                    bool three = false);

int launch_row_fwd(const RowProblem &p, hipStream_t st);
int launch_row_bwd(const RowProblem &p, hipStream_t st);
size_t row_bwd_workspace_bytes(int mode, int64_t rows, int64_t R, int64_t planes);

struct BnProblem {
  int dtype = 0;
  const void *x = nullptr;
  const void *dy = nullptr;
  void *out = nullptr; // y or dx
  const float *gamma = nullptr;
  const float *beta = nullptr;
  float *batch_mean = nullptr; // forward: written
  float *batch_var = nullptr;
  float *rmean = nullptr;
  float *rvar = nullptr;
  const float *mean = nullptr; // backward / inference: read
  const float *var = nullptr;
  const float *dmean = nullptr;
  const float *dvar = nullptr;
  float *dgamma = nullptr;
  float *dbeta = nullptr;
  int accum_dx = 0, accum_g = 0, accum_b = 0;
  int batch_stat = 1;
  // FusedBatchNormalization: forward y = max(0, bn(x) [+ z]) when relu != 0;
  // backward masks dy by y > 0 when y != null and writes the masked dy to dz.
  int relu = 0;
  const void *z = nullptr;
  const void *y = nullptr;
  void *dz = nullptr;
  int accum_dz = 0;
  // Split-batch (SyncBatchNormalization) steps: backward pair sums out
  // ([C][2] = sum dy*(x-mean), sum dy), or in together with the total count.
  float *sums_out = nullptr;
  const float *sums_in = nullptr;
  double total_count = 0.0;
  int64_t size0 = 1, C = 1, size2 = 1;
  float decay = 0.9f, eps = 1e-5f;
  void *ws = nullptr;
  size_t ws_bytes = 0;
};

// BatchNormalization training forward / backward with a channel cached in
// registers (one launch, x and dy cross HBM once per direction): false when
// the shape or the flags are not theirs, else *status holds the launch result.
bool bn_rows_fwd_train(const BnProblem &p, hipStream_t st, int *status);
// Training forward with a channel of up to 25600 vectors held on one CU
// (registers and LDS), for tensors with a channel per CU (bn_onchip.hip).
bool bn_onchip_fwd_train(const BnProblem &p, hipStream_t st, int *status);
// ... and the backward with x held there and dy streamed past it twice.
bool bn_onchip_bwd(const BnProblem &p, hipStream_t st, int *status);
bool bn_rows_bwd(const BnProblem &p, hipStream_t st, int *status);
// The same for channel-last tensors of few rows (gn_cl_rows.hip): a block per
// channel vector keeps its column in registers.
bool bn_cl_cached_fwd_train(const BnProblem &p, hipStream_t st, int *status);
// Channel-last training forward with the whole tensor held on the chip's CUs
// and the per-channel partials exchanged between the blocks (bn_cl_grid.hip).
bool bn_cl_grid_fwd_train(const BnProblem &p, hipStream_t st, int *status);
bool bn_cl_grid_bwd(const BnProblem &p, hipStream_t st, int *status);
bool bn_cl_cached_bwd(const BnProblem &p, hipStream_t st, int *status);
// Training forward / backward for planes that are not a whole number of
// 16-byte vectors (7x7, half 14x14): a pack of 2, 4 or 8 neighbouring channels,
// whose planes together are, held on one CU (bn_pack.hip).
// Channel-last training forward / backward of up to 65536 rows through the
// split kernels of gn_cl_split.hip (all rows as one sample, a unit per channel).
bool bn_cl_split_fwd_train(const BnProblem &p, hipStream_t st, int *status);
bool bn_cl_split_bwd(const BnProblem &p, hipStream_t st, int *status);
// Training forward / backward for fewer channels than CUs: a channel split
// over 2 - 8 blocks that hold their samples on chip and exchange partial sums
// (bn_split_channel.hip).
bool bn_chan_split_fwd_train(const BnProblem &p, hipStream_t st, int *status);
bool bn_chan_split_bwd(const BnProblem &p, hipStream_t st, int *status);
// Planes that are no whole number of vectors, a channel held by one block
// (rows_masked.hip); false: not taken.
bool bn_masked_fwd_train(const BnProblem &p, hipStream_t st, int *status);
// Whether the masked kernels (a block per channel) would take this problem.
bool bn_masked_takes(const BnProblem &p, bool backward);
bool bn_masked_bwd(const BnProblem &p, hipStream_t st, int *status);
bool bn_pack_fwd_train(const BnProblem &p, hipStream_t st, int *status);
bool bn_pack_bwd(const BnProblem &p, hipStream_t st, int *status);
int launch_bn_infer(const BnProblem &p, hipStream_t st);
int launch_bn_fwd_train(const BnProblem &p, hipStream_t st);
int launch_bn_bwd(const BnProblem &p, hipStream_t st);
// Local statistics only (p.out unused), merge of per-shard statistics, and the
// backward apply step from summed pairs (p.sums_in, p.total_count).
int launch_bn_local_stats(const BnProblem &p, hipStream_t st);
int launch_bn_merge_stats(const float *stats, int workers, int64_t C, float *batch_mean,
                          float *batch_var, float *rmean, float *rvar, float decay,
                          hipStream_t st);
int launch_bn_bwd_from_sums(const BnProblem &p, hipStream_t st);
// out[i] = in[0][i] + in[1][i] + ... + in[rows-1][i], i < n (rows in order).
int launch_sum_rows(const float *in, int rows, int64_t n, float *out, hipStream_t st);
size_t bn_workspace_bytes(int64_t size0, int64_t C, int64_t size2, int dtype);

// Optional per-kernel timing.  When enabled, a launch goes through
// hipExtLaunchKernelGGL with a start/stop event pair, which stamps the
// kernel's own dispatch (begin and end of execution on the device), the same
// interval a kernel trace reports.  Off by default; see nblahip_profile_* in
// the C-ABI.  Returns false (and leaves the events untouched) when timing is
// off or the pool is exhausted.
bool prof_acquire(const char *tag, hipEvent_t *start, hipEvent_t *stop);

#define NBLAHIP_LAUNCH(tag, kern, grid, block, shmem, st, ...)                          \
  do {                                                                                  \
    hipEvent_t prof_ev0_, prof_ev1_;                                                    \
    if (::nblahip::prof_acquire(tag, &prof_ev0_, &prof_ev1_)) {                         \
      hipExtLaunchKernelGGL(kern, grid, block, shmem, st, prof_ev0_, prof_ev1_, 0,      \
                            __VA_ARGS__);                                               \
    } else {                                                                            \
      hipLaunchKernelGGL(kern, grid, block, shmem, st, __VA_ARGS__);                    \
    }                                                                                   \
  } while (0)

// Channel-last Group/InstanceNormalization: x is [batch, spatial, channels].
struct ClProblem {
  int dtype = 0;
  const void *x = nullptr;
  const void *dy = nullptr;
  void *out = nullptr; // y or dx
  const float *gamma = nullptr;
  const float *beta = nullptr;
  float *mean = nullptr; // [batch*groups], forward: written; backward: read
  float *var = nullptr;
  const float *dmean = nullptr;
  const float *dvar = nullptr;
  float *dgamma = nullptr;
  float *dbeta = nullptr;
  int accum_dx = 0, accum_g = 0, accum_b = 0;
  int64_t batch = 1, spatial = 1, channels = 1;
  int groups = 1;
  int bc_gamma = 1, bc_beta = 1; // parameters shared by the batch (always for groups)
  float eps = 0.f;
  void *ws = nullptr;
  size_t ws_bytes = 0;
  // Channel-last BatchNormalization through the split kernels (one "sample" of
  // all rows, a unit per channel): the running statistics to update, may be null.
  float *rmean = nullptr;
  float *rvar = nullptr;
  float decay = 0.f, unbias = 1.f;
  int as_batch_norm = 0;
};
// Register-cached channel-last GroupNormalization (gn_cl_rows.hip): false when
// the shape is not theirs, else *status holds the launch result.  The backward
// leaves the per-(n, channel) pairs in `pairs` for the batch sum.
bool gn_cl_cached_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status);
bool gn_cl_cached_bwd(const ClProblem &p, bool aligned, float *pairs, hipStream_t st, int *status);
// Split channel-last kernels (gn_cl_split.hip): a block owns whole 128-byte
// lines of a position range, the blocks of a sample exchange partial sums.  The
// backward leaves per-block pairs in the workspace: *pairs is [*pair_batches][C][2].
constexpr int kClSplitMaxBlocks = 64; // blocks per (sample, column tile), i.e. pairs per channel
bool cl_split_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status);
bool cl_split_bwd(const ClProblem &p, bool aligned, float **pairs, int64_t *pair_batches,
                  hipStream_t st, int *status);
// Channel-last GroupNormalization with groups that are no whole number of
// vectors (gn_cl_tile.hip): a block owns whole rows of a position range, the
// blocks of a sample exchange per-group partial sums.  The backward leaves
// per-block pairs in the workspace like cl_split_bwd.
bool cl_tile_fwd(const ClProblem &p, bool aligned, hipStream_t st, int *status);
bool cl_tile_bwd(const ClProblem &p, bool aligned, float **pairs, int64_t *pair_batches,
                 hipStream_t st, int *status);
int launch_cl_fwd(const ClProblem &p, hipStream_t st);
int launch_cl_bwd(const ClProblem &p, hipStream_t st);
size_t cl_workspace_bytes(int64_t batch, int64_t spatial, int64_t channels, int dtype);

inline int last_launch_status() {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : static_cast<int>(e);
}

} // namespace nblahip
