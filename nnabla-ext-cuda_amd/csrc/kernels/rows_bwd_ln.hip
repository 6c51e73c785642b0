// Instantiations and launcher of the register-cached backward row kernel,
// mode kRowLN.
#include <map>
#include <mutex>
#include <tuple>

#include "rows_dispatch.hpp"

namespace nblahip {

// The layouts pick_ln_bwd_cfg hands out (rows_host.hip), and no others: up to
// four vectors per thread (the per-column accumulators make every load cost
// about 27 registers: eight of them spill 600 - 1200 bytes per lane), one per
// thread at 1024 threads - two for float.
#define LN_CASES_TPR(CASE, T, VEC, TPR) CASE(T, VEC, 1, TPR) CASE(T, VEC, 2, TPR) CASE(T, VEC, 4, TPR)
#define LN_CASES_VEC(CASE, T, VEC)                                                     \
  NBLAHIP_ROW_CASES_SUBWAVE(CASE, T, VEC)                                              \
  LN_CASES_TPR(CASE, T, VEC, 64)                                                       \
  LN_CASES_TPR(CASE, T, VEC, 256)                                                      \
  LN_CASES_TPR(CASE, T, VEC, 512)                                                      \
  CASE(T, VEC, 1, 1024)
#define LN_CASES(CASE, T)                                                              \
  LN_CASES_VEC(CASE, T, FullVec<T>::value)                                             \
  CASE(T, FullVec<T>::value, 3, 64)                                                    \
  CASE(T, FullVec<T>::value, 3, 256)                                                   \
  CASE(T, FullVec<T>::value, 3, 512)                                                   \
  LN_CASES_VEC(CASE, T, MidVec<T>::value)                                              \
  LN_CASES_VEC(CASE, T, 1)                                                             \
  if constexpr (sizeof(T) == 4) {                                                      \
    CASE(T, FullVec<T>::value, 2, 1024)                                                \
    CASE(T, 1, 2, 1024)                                                                \
  }

// Layouts that exist with the next row asked for ahead: a block per row, two
// or three of the widest vectors per thread in half, three at 512 threads in
// float (ln_bwd_rows_ahead in rows_host.hip has the measurements).
template <typename T, int VEC, int NL, int TPR>
constexpr bool kBwdAhead = VEC == FullVec<T>::value &&
                           (sizeof(T) == 2 ? (NL == 2 || NL == 3) && (TPR == 256 || TPR == 512)
                                           : NL == 3 && TPR == 512);

#define BWD_CASE(T, VEC, NL, TPR)                                                      \
  if (cfg.vec == (VEC) && cfg.nl == (NL) && cfg.tpr == (TPR)) {                        \
    if constexpr (kBwdAhead<T, VEC, NL, TPR>) {                                        \
      if (cfg.ahead) {                                                                 \
        NBLAHIP_LAUNCH("row_bwd_kernel_ln", (row_bwd_kernel<T, VEC, NL, TPR, kRowLN, true>),             \
                       dim3(grid), dim3(RowBwdBlock<TPR, kRowLN>::kBlock), 0, st, args);                \
        return last_launch_status();                                                   \
      }                                                                                \
    }                                                                                  \
    NBLAHIP_LAUNCH("row_bwd_kernel_ln", (row_bwd_kernel<T, VEC, NL, TPR, kRowLN>), dim3(grid),           \
                       dim3(RowBwdBlock<TPR, kRowLN>::kBlock), 0, st, args);                      \
    return last_launch_status();                                                       \
  }

template <typename T>
static int run_bwd_t(const RowCfg &cfg, const RowArgs &args, int grid, hipStream_t st) {
  LN_CASES(BWD_CASE, T)
  return NBLAHIP_EINVAL;
}

// Blocks of the selected kernel that fit one CU at the same time (register and
// LDS use decide), asked of the runtime once per layout: the persistent grid
// of the LayerNormalization backward should fill the chip in one round.
#define OCC_CASE(T, VEC, NL, TPR)                                                      \
  if (cfg.vec == (VEC) && cfg.nl == (NL) && cfg.tpr == (TPR)) {                        \
    int n = 0;                                                                         \
    if constexpr (kBwdAhead<T, VEC, NL, TPR>) {                                        \
      if (cfg.ahead) {                                                                 \
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(                              \
                &n, row_bwd_kernel<T, VEC, NL, TPR, kRowLN, true>,                     \
                RowBwdBlock<TPR, kRowLN>::kBlock, 0) != hipSuccess)                    \
          n = 0;                                                                       \
        return n;                                                                      \
      }                                                                                \
    }                                                                                  \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(                                  \
            &n, row_bwd_kernel<T, VEC, NL, TPR, kRowLN>,                               \
            RowBwdBlock<TPR, kRowLN>::kBlock, 0) != hipSuccess)                        \
      n = 0;                                                                           \
    return n;                                                                          \
  }

template <typename T> static int occupancy_t(const RowCfg &cfg) {
  LN_CASES(OCC_CASE, T)
  return 0;
}

int row_bwd_ln_resident_blocks(int dtype, const RowCfg &cfg) {
  static std::mutex mu;
  static std::map<std::tuple<int, int, int, int, bool>, int> cache;
  const auto key = std::make_tuple(dtype, cfg.vec, cfg.nl, cfg.tpr, cfg.ahead);
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it == cache.end()) {
    const int n = dtype == NBLAHIP_F16 ? occupancy_t<__half>(cfg) : occupancy_t<float>(cfg);
    it = cache.emplace(key, n).first;
  }
  return it->second;
}

int run_row_bwd_cached_ln(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st) {
  return dtype == NBLAHIP_F16 ? run_bwd_t<__half>(cfg, args, grid, st)
                              : run_bwd_t<float>(cfg, args, grid, st);
}

} // namespace nblahip
