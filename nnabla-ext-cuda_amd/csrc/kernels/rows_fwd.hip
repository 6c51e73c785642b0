// Instantiations and launcher of the register-cached forward row kernel.
#include "rows_dispatch.hpp"

namespace nblahip {

// Layouts that exist with the next row asked for ahead (widest vector, a wave
// or a block of up to 512 threads per row, at most four loads per thread).
template <typename T, int VEC, int NL, int TPR>
constexpr bool kRowsAhead = VEC == FullVec<T>::value && TPR >= 64 && TPR <= 512 && NL <= 4;

#define FWD_CASE(T, VEC, NL, TPR)                                                      \
  if (cfg.vec == (VEC) && cfg.nl == (NL) && cfg.tpr == (TPR)) {                        \
    if (args.percol) {                                                                 \
      if constexpr (kRowsAhead<T, VEC, NL, TPR>) {                                     \
        if (args.ahead) {                                                              \
          NBLAHIP_LAUNCH("row_fwd_kernel", (row_fwd_kernel<T, VEC, NL, TPR, true, false, true>), \
                         dim3(grid), dim3(RowBlock<TPR>::kBlock), 0, st, args);        \
          return last_launch_status();                                                 \
        }                                                                              \
      }                                                                                \
      NBLAHIP_LAUNCH("row_fwd_kernel", (row_fwd_kernel<T, VEC, NL, TPR, true>), dim3(grid), \
                     dim3(RowBlock<TPR>::kBlock), 0, st, args);                        \
    } else {                                                                           \
      NBLAHIP_LAUNCH("row_fwd_kernel", (row_fwd_kernel<T, VEC, NL, TPR, false>), dim3(grid), \
                     dim3(RowBlock<TPR>::kBlock), 0, st, args);                        \
    }                                                                                  \
    return last_launch_status();                                                       \
  }

template <typename T>
static int run_fwd_t(const RowCfg &cfg, const RowArgs &args, int grid, hipStream_t st) {
  NBLAHIP_ROW_CASES(FWD_CASE, T)
  NBLAHIP_ROW_CASES_THREE(FWD_CASE, T)
  return NBLAHIP_EINVAL;
}

int run_row_fwd_cached(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                       hipStream_t st) {
  return dtype == NBLAHIP_F16 ? run_fwd_t<__half>(cfg, args, grid, st)
                              : run_fwd_t<float>(cfg, args, grid, st);
}

} // namespace nblahip
