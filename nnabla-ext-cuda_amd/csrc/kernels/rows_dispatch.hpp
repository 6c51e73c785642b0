// Internal: per-family launchers of the register-cached row kernels.  Each
// lives in its own translation unit so the template instantiations compile
// in parallel.
#pragma once

#include "launch.hpp"
#include "rows.cuh"

namespace nblahip {

int run_row_fwd_cached(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                       hipStream_t st);
// A row of up to 400 KB held on one CU (registers + LDS), GroupNormalization and
// InstanceNormalization forward; false: not taken.
bool row_onchip_fwd(const RowProblem &p, const RowArgs &args, int vec, hipStream_t st, int *status);
// InstanceNormalization planes that are no whole number of 16-byte vectors, with
// 16-byte loads over the tensor's aligned vectors; false: not taken.
bool row_masked_fwd(const RowProblem &p, hipStream_t st, int *status);
bool row_masked_bwd(const RowProblem &p, hipStream_t st, int *status); // the pairs to p.ws
int run_row_bwd_cached_ln(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st);
// LayerNormalization backward over rows that are no whole number of 16-byte
// vectors or start off a 16-byte boundary, with 16-byte accesses at element
// alignment (rows_ln_loose.hip).  wanted: the problem is one of these (vec: the
// width the aligned layouts would use); cfg: a wave-per-row layout of full
// vectors for the row length rounded up to whole vectors.
bool ln_loose_bwd_wanted(const RowProblem &p, int vec);
int ln_loose_bwd(const RowProblem &p, const RowArgs &a, const RowCfg &cfg, int grid, hipStream_t st);
// Resident blocks per CU of the LayerNormalization backward kernel for cfg
// (0 when the runtime cannot tell).
int row_bwd_ln_resident_blocks(int dtype, const RowCfg &cfg);
int run_row_bwd_cached_in(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st);
int run_row_bwd_cached_inc(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                           hipStream_t st);
int run_row_bwd_cached_gn(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st);
int run_row_fwd_cached_bn(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st);
int run_row_bwd_cached_bn(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                          hipStream_t st);
int run_row_bwd_cached_lnx(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                           hipStream_t st);
int run_row_bwd_cached_gnm(int dtype, const RowCfg &cfg, const RowArgs &args, int grid,
                           hipStream_t st);

// Expands CASE(T, VEC, NL, TPR) for every supported register-cached shape of
// element type T (for float the MidVec lines repeat the FullVec ones: same
// instantiations, unreachable branches).
#define NBLAHIP_ROW_CASES_TPR(CASE, T, VEC, TPR) \
  CASE(T, VEC, 1, TPR) CASE(T, VEC, 2, TPR) CASE(T, VEC, 4, TPR) CASE(T, VEC, 8, TPR)

// Three loads per thread with the widest vector: rows of 3 x 2^k vectors (hidden
// sizes 768, 1536, 3072, 6144, 12288) exactly, 5 x 2^k (2560, 5120) at 83 %.
#define NBLAHIP_ROW_CASES_THREE(CASE, T)                                          \
  CASE(T, FullVec<T>::value, 3, 64) CASE(T, FullVec<T>::value, 3, 256)            \
  CASE(T, FullVec<T>::value, 3, 512) CASE(T, FullVec<T>::value, 3, 1024)

// Rows of a few hundred bytes: several rows per wave, at most 4 loads each.
#define NBLAHIP_ROW_CASES_SUBWAVE(CASE, T, VEC)                                   \
  CASE(T, VEC, 1, 4) CASE(T, VEC, 2, 4) CASE(T, VEC, 4, 4)                        \
  CASE(T, VEC, 1, 8) CASE(T, VEC, 2, 8) CASE(T, VEC, 4, 8)                        \
  CASE(T, VEC, 1, 16) CASE(T, VEC, 2, 16) CASE(T, VEC, 4, 16)                     \
  CASE(T, VEC, 1, 32) CASE(T, VEC, 2, 32) CASE(T, VEC, 4, 32)

#define NBLAHIP_ROW_CASES(CASE, T)                          \
  NBLAHIP_ROW_CASES_SUBWAVE(CASE, T, FullVec<T>::value)     \
  NBLAHIP_ROW_CASES_SUBWAVE(CASE, T, MidVec<T>::value)      \
  NBLAHIP_ROW_CASES_SUBWAVE(CASE, T, 1)                     \
  NBLAHIP_ROW_CASES_WAVE(CASE, T)

// One wave or more per row.
#define NBLAHIP_ROW_CASES_WAVE(CASE, T)                     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 64)     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 256)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 512)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 1024)   \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 64)      \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 256)     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 512)     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 1024)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 64)                     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 256)                    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 512)                    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 1024)

#define NBLAHIP_ROW_CASES_BLOCK(CASE, T)                    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 256)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 512)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, FullVec<T>::value, 1024)   \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 256)     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 512)     \
  NBLAHIP_ROW_CASES_TPR(CASE, T, MidVec<T>::value, 1024)    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 256)                    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 512)                    \
  NBLAHIP_ROW_CASES_TPR(CASE, T, 1, 1024)

} // namespace nblahip
