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

template <typename T>
static int run_bwd_t(const RowCfg &cfg, const RowArgs &args, int grid, hipStream_t st) {
  NBLAHIP_ROW_CASES_BLOCK(BWD_CASE, T)
  return NBLAHIP_EINVAL;
}

int run_row_bwd_cached_lnx(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st) {
  return dtype == NBLAHIP_F16 ? run_bwd_t<__half>(cfg, args, grid, st)
                              : run_bwd_t<float>(cfg, args, grid, st);
}

} // namespace nblahip
