// FusedBatchNormalization instantiations of the cached channel-last instance
// kernels (channel-last tensors of few rows).
#include "gn_cl_rows.cuh"

namespace nblahip {

#define FUSED_CASES_TPR(CASE, T, VEC, TPR) \
  CASE(T, VEC, 1, TPR) CASE(T, VEC, 2, TPR) CASE(T, VEC, 4, TPR) CASE(T, VEC, 8, TPR)
#define FUSED_CASES(CASE, T, VEC)                                        \
  FUSED_CASES_TPR(CASE, T, VEC, 64) FUSED_CASES_TPR(CASE, T, VEC, 256)   \
  FUSED_CASES_TPR(CASE, T, VEC, 512) FUSED_CASES_TPR(CASE, T, VEC, 1024)

// The backward takes planes of up to 2048 positions (pick_in_cfg), which the
// wave and the 256-thread layouts hold: the larger blocks are never picked.
#define FUSED_CASES_BWD(CASE, T, VEC) FUSED_CASES_TPR(CASE, T, VEC, 64) FUSED_CASES_TPR(CASE, T, VEC, 256)

#define FWD_CASE(T, VEC, NL, TPR)                                                                \
  if (nl == (NL) && tpr == (TPR)) {                                                              \
    if (fuse == 2) {                                                                             \
      NBLAHIP_LAUNCH("in_cl_row_fwd_kernel_fused", (in_cl_row_fwd_kernel<T, VEC, NL, TPR, 2>),   \
                     dim3(grid), dim3(TPR), 0, st, a);                                           \
    } else {                                                                                     \
      NBLAHIP_LAUNCH("in_cl_row_fwd_kernel_fused", (in_cl_row_fwd_kernel<T, VEC, NL, TPR, 1>),   \
                     dim3(grid), dim3(TPR), 0, st, a);                                           \
    }                                                                                            \
    return last_launch_status();                                                                 \
  }
#define BWD_CASE(T, VEC, NL, TPR)                                                                \
  if (nl == (NL) && tpr == (TPR)) {                                                              \
    NBLAHIP_LAUNCH("in_cl_row_bwd_kernel_fused", (in_cl_row_bwd_kernel<T, VEC, NL, TPR, true>),  \
                   dim3(grid), dim3(TPR), 0, st, a);                                             \
    return last_launch_status();                                                                 \
  }

int run_in_fwd_fused(int dtype, int tpr, int nl, const GnClArgs &a, unsigned grid, int fuse,
                     hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    FUSED_CASES(FWD_CASE, __half, 8)
  } else {
    FUSED_CASES(FWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

int run_in_bwd_fused(int dtype, int tpr, int nl, const GnClArgs &a, unsigned grid, hipStream_t st) {
  if (dtype == NBLAHIP_F16) {
    FUSED_CASES_BWD(BWD_CASE, __half, 8)
  } else {
    FUSED_CASES_BWD(BWD_CASE, float, 4)
  }
  return NBLAHIP_EINVAL;
}

} // namespace nblahip
