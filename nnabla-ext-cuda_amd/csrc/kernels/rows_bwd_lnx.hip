// Instantiations and launcher of the register-cached backward row kernel,
// mode kRowLNx (dx of long LayerNormalization rows).
#include "rows_dispatch.hpp"

namespace nblahip {

#define BWD_CASE(T, VEC, NL, TPR)                                                      \
  if (cfg.vec == (VEC) && cfg.nl == (NL) && cfg.tpr == (TPR)) {                        \
    NBLAHIP_LAUNCH("row_bwd_kernel_lnx", (row_bwd_kernel<T, VEC, NL, TPR, kRowLNx>), dim3(grid),           \
                       dim3(RowBwdBlock<TPR, kRowLNx>::kBlock), 0, st, args);                      \
    return last_launch_status();                                                       \
  }

// This mode takes the rows beyond the layouts of the plain LayerNormalization
// backward (more than 2048 vectors), for which pick_row_cfg (rows_host.hip:
// eight vectors per thread below 1024 threads, four - scalar rows: eight - at
// 1024) has these layouts left.
template <typename T>
static int run_bwd_t(const RowCfg &cfg, const RowArgs &args, int grid, hipStream_t st) {
  BWD_CASE(T, FullVec<T>::value, 8, 512)
  BWD_CASE(T, MidVec<T>::value, 8, 512)
  BWD_CASE(T, 1, 8, 512)
  BWD_CASE(T, FullVec<T>::value, 4, 1024)
  BWD_CASE(T, MidVec<T>::value, 4, 1024)
  BWD_CASE(T, 1, 4, 1024)
  BWD_CASE(T, 1, 8, 1024)
  return NBLAHIP_EINVAL;
}

int run_row_bwd_cached_lnx(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st) {
  return dtype == NBLAHIP_F16 ? run_bwd_t<__half>(cfg, args, grid, st)
                              : run_bwd_t<float>(cfg, args, grid, st);
}

} // namespace nblahip
