// GroupNormalization / InstanceNormalization forward for rows beyond what a
// block's registers alone hold (128 KB) with the row held on one CU all the
// same: NR 16-byte vectors per thread in registers, NS more in LDS (each
// thread reads back what it wrote).  One 1024-thread block per row reads it
// once, reduces, and writes y: 2 S where the streaming kernels move 3 S.
// NR + NS = 25 covers rows of 400 KB: float groups of 100 k elements
// ([N,320,64,64] in 32 groups, 256x256 planes), half groups of 200 k.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"
#include "onchip.cuh"
#include "rows.cuh"

namespace nblahip {

// OVER: the row is longer than the NR + NS slots.  The rest is read once for
// the statistics (into the same per-thread sums as the held part) and a second
// time for y: 2 S + (1 - 25600 / nv) S.
template <typename T, int VEC, int NR, int NS, bool OVER = false>
__global__ void __launch_bounds__(kOnchipBlock)
row_onchip_fwd_kernel(const RowArgs a) {
  static_assert(sizeof(RawVec<T, VEC>) == 16, "16-byte vectors");
  __shared__ float red[kOnchipBlock / kWave];
  __shared__ uint4 spill[NS > 0 ? NS * kOnchipBlock : 1];
  const uint32_t row = blockIdx.x;
  const uint32_t t = threadIdx.x;
  const uint32_t nv = static_cast<uint32_t>(a.R) / VEC;
  const T *__restrict__ x = static_cast<const T *>(a.x) + static_cast<size_t>(row) * a.R;
  T *__restrict__ y = static_cast<T *>(a.out) + static_cast<size_t>(row) * a.R;

  // All loads in flight together, without a branch: a slot beyond the row
  // reads the row's last vector and is left out of every sum and store.  The
  // LDS part first: its registers are free again once the values are parked.
  RawVec<T, VEC> parked[NS > 0 ? NS : 1];
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t;
    parked[k] = load_raw<T, VEC>(x + min(v, nv - 1u) * VEC);
  }
  RawVec<T, VEC> raw[NR];
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t;
    raw[k] = load_raw<T, VEC>(x + min(v, nv - 1u) * VEC);
  }
  // Statistics from sums every wave takes over its OWN registers as its loads
  // arrive (the memory system serves a CU's waves one after the other: what a
  // wave does before the block's first barrier hides behind the other waves'
  // loads, a second pass about the row's mean would keep memory idle).  Per
  // thread: s = sum x, then about the thread's own mean K = s / n:
  // s1 = sum (x - K) (rounding residue), s2 = sum (x - K)^2; mean = sum_t s / R
  // and, about it, var = sum_t (s2 + 2 e s1 + n e^2) / R with e = K - mean: two
  // block sums of a few operations per thread.  sum_t n e^2 is the variance
  // between the threads' means, never more than the total: nothing cancels.
  // (OVER: the vectors beyond the held ones are read here once, shifted by the
  // K of the thread's held elements, and once more for y.)
  auto held = [&](int k) { return static_cast<int>(t) < static_cast<int>(nv) - k * kOnchipBlock; };
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const float part = raw_sum<T, VEC>(parked[k], 0.f);
    s += held(NR + k) ? part : 0.f;
    spill[k * kOnchipBlock + t] = __builtin_bit_cast(uint4, parked[k]);
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const float part = raw_sum<T, VEC>(raw[k], 0.f);
    s += held(k) ? part : 0.f;
  }
  constexpr uint32_t kHeld = static_cast<uint32_t>(NR + NS) * kOnchipBlock;
  const uint32_t nvh = OVER ? min(nv, kHeld) : nv; // held vectors of the row
  const float nh = t < nvh ? static_cast<float>(((nvh - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
  const float kk = s * (1.0f / fmaxf(nh, 1.f));
  float s1 = 0.f, s2 = 0.f;
  auto take = [&](const RawVec<T, VEC> &r) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = elem_fma<T, VEC>(r, j, a.one, -kk);
      s1 += d;
      s2 = fmaf(d, d, s2);
    }
  };
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    if (held(NR + k)) take(parked[k]);
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    if (held(k)) take(raw[k]);
  }
  float nt = nh; // elements of the thread, held and streamed
  constexpr int BO = 4; // vectors per thread and step of the streamed rest
  if constexpr (OVER) {
#pragma unroll 1
    for (uint32_t v0 = kHeld; v0 < nv; v0 += BO * kOnchipBlock) {
      RawVec<T, VEC> xo[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b)
        xo[b] = load_raw<T, VEC>(x + min(v0 + b * kOnchipBlock + t, nv - 1u) * VEC);
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        if (v0 + b * kOnchipBlock + t < nv) take(xo[b]);
      }
    }
    nt = t < nv ? static_cast<float>(((nv - 1u - t) / kOnchipBlock + 1u) * VEC) : 0.f;
  }
  // (n K + s1 = the thread's sum of x, held and streamed)
  const float mean = onchip_block_sum(fmaf(nt, kk, s1), red) * a.inv_R;
  const float e = kk - mean;
  const float var = onchip_block_sum(fmaf(e, fmaf(nt, e, 2.f * s1), s2), red) * a.inv_R;
  const float istd = inv_std(var, a.eps);
  if (t == 0) {
    a.mean[row] = mean;
    a.var[row] = var;
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) keep_packed<T, VEC>(raw[k]);

  // gamma/beta of a vector: one channel (a plane is a whole number of vectors)
  const uint32_t pbase = (row % a.pmod) * a.pmul;
  const uint32_t bbase = (row % a.pmod_b) * a.pmul;
  auto emit = [&](const RawVec<T, VEC> &r, uint32_t v) {
    const uint32_t poff = a.pdiv.div(v * VEC);
    const float g = (a.gamma ? a.gamma[pbase + poff] : 1.f) * istd;
    const float b = a.beta ? a.beta[bbase + poff] : 0.f;
    float o[VEC];
    if constexpr (sizeof(T) == 2) {
      const float sh = fmaf(-mean, g, b); // x*g + (b - mean*g): one mixed fma, rounded once
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = elem_fma<T, VEC>(r, j, g, sh);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = fmaf(elem_fma<T, VEC>(r, j, a.one, -mean), g, b);
    }
    store_vec<T, VEC>(y + v * VEC, o);
  };
  const uint32_t t2 = fresh(t);
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kOnchipBlock + t2;
    if (v < nv) emit(raw[k], v);
  }
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const uint32_t v = static_cast<uint32_t>(NR + k) * kOnchipBlock + t2;
    if (v < nv) emit(__builtin_bit_cast(RawVec<T, VEC>, spill[k * kOnchipBlock + t]), v);
  }
  if constexpr (OVER) {
#pragma unroll 1
    for (uint32_t v0 = kHeld; v0 < nv; v0 += BO * kOnchipBlock) {
      RawVec<T, VEC> xo[BO];
#pragma unroll
      for (int b = 0; b < BO; ++b)
        xo[b] = load_raw<T, VEC>(x + min(v0 + b * kOnchipBlock + t, nv - 1u) * VEC);
#pragma unroll
      for (int b = 0; b < BO; ++b) {
        const uint32_t v = v0 + b * kOnchipBlock + t;
        if (v < nv) emit(xo[b], v);
      }
    }
  }
}

namespace {

template <typename T, int VEC>
int run_onchip_fwd(int nl, const RowArgs &a, int grid, hipStream_t st) {
#define ONCHIP_ROW_FWD(NR, NS)                                                              \
  if (nl <= (NR) + (NS)) {                                                                  \
    NBLAHIP_LAUNCH("row_onchip_fwd_kernel", (row_onchip_fwd_kernel<T, VEC, NR, NS>),        \
                   dim3(grid), dim3(kOnchipBlock), 0, st, a);                               \
    return last_launch_status();                                                            \
  }
  ONCHIP_ROW_FWD(10, 0)
  ONCHIP_ROW_FWD(12, 0)
  ONCHIP_ROW_FWD(14, 0)
  ONCHIP_ROW_FWD(16, 0)
  ONCHIP_ROW_FWD(16, 3)
  ONCHIP_ROW_FWD(16, 6)
  ONCHIP_ROW_FWD(16, 9)
#undef ONCHIP_ROW_FWD
  // longer rows: 25 slots held, the rest streamed
  NBLAHIP_LAUNCH("row_onchip_fwd_kernel", (row_onchip_fwd_kernel<T, VEC, 16, 9, true>), dim3(grid),
                 dim3(kOnchipBlock), 0, st, a);
  return last_launch_status();
}

} // namespace

// Rows of 4097..25600 full vectors (from 64 KB on it also beats the row kernels
// that hold such a row in 8 vectors per thread: 80 KB half groups 18.0 -> 14.0
// us, 120 KB 24.4 -> 19.7 us, float 80 KB 17.3 -> 13.4 us, 128 KB half planes
// 25.6 -> 21.0 us; 64 KB: 12.2 either way), at least an eighth as many as there are
// CUs (the block is alone on its CU; with fewer rows the streaming kernels,
// which split a row over many blocks, use more of the chip: 32 groups of 160 KB
// 8.3 vs 11.8 us, 16 of 320 KB 12.6 vs 11.7 us); up to 65536 vectors with the
// first 25600 held, given a row for nearly every CU.
bool row_onchip_fwd(const RowProblem &p, const RowArgs &a, int vec, hipStream_t st, int *status) {
  if (!tune_int("ROW_ONCHIP", 1)) return false;
  if (p.mode == kRowLN || !p.out) return false;
  if (vec != (p.dtype == NBLAHIP_F16 ? 8 : 4)) return false;
  const int64_t nv = p.R / vec;
  if (nv < tune_int("ROW_ONCHIP_FWD_MIN_VECTORS", 4097) || nv > 65536) return false;
  // Rows that one block's registers hold as well (up to 8192 vectors) want
  // rows for an eighth of the CUs (fewer: [1,C,256,256] half 21.8 vs 20.5 us at
  // C = 24); longer ones, which otherwise stream, win from the first row
  // ([1,C,512,256] half forward + backward 34.8 vs 42.7 us at C = 4, 33.9 vs
  // 43.1 at 24; [1,C,256,256] float 28.6 vs 37.7 at 4, 27.8 vs 38.0 at 24).
  const int min_pct = nv <= 25 * kOnchipBlock
                          ? tune_int("ROW_ONCHIP_MIN_PCT", nv <= 8 * kOnchipBlock ? 12 : 1)
                          : tune_int("ROW_ONCHIP_STREAMED_MIN_PCT", 88);
  if (p.rows * 100 < static_cast<int64_t>(device_cus()) * min_pct) return false;
  const int nl = static_cast<int>((nv + kOnchipBlock - 1) / kOnchipBlock);
  const int grid = static_cast<int>(p.rows);
  *status = p.dtype == NBLAHIP_F16 ? run_onchip_fwd<__half, 8>(nl, a, grid, st)
                                   : run_onchip_fwd<float, 4>(nl, a, grid, st);
  return true;
}

} // namespace nblahip
