// Second stage of the Instance/GroupNormalization parameter gradients:
// pairs[n][P][2] holds (dgamma part, dbeta part) per sample and parameter.
// A parameter shared by the batch gets the sum over n, a per-sample parameter
// its own pair.  Templates so that the translation units that launch them
// (rows and channel-last paths) can both include this header.
#pragma once

#include "common.cuh"
#include "launch.hpp"

namespace nblahip {

// Sum over the batch.  A block covers 256 / TY adjacent parameters; its TY
// thread rows take the samples ty, ty + TY, ... (8 independent loads in
// flight), then fold in row order through LDS, so the result does not depend
// on the grid.  Either output may be null.
template <int TY>
__global__ void __launch_bounds__(256)
pair_batch_sum_kernel(const float *__restrict__ pairs, int n, int P,
                      float *__restrict__ dgamma, float *__restrict__ dbeta, int accum_g,
                      int accum_b) {
  constexpr int TX = 256 / TY;
  __shared__ float fold_g[256];
  __shared__ float fold_b[256];
  const int tx = threadIdx.x % TX;
  const int ty = threadIdx.x / TX;
  const int i = blockIdx.x * TX + tx;
  const float2 *__restrict__ pp = reinterpret_cast<const float2 *>(pairs);
  float sg = 0.f, sb = 0.f;
  if (i < P) {
    for (int b0 = ty; b0 < n; b0 += TY * 8) {
      float2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int b = b0 + u * TY;
        v[u] = (b < n) ? pp[static_cast<size_t>(b) * P + i] : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        sg += v[u].x;
        sb += v[u].y;
      }
    }
  }
  fold_g[ty * TX + tx] = sg;
  fold_b[ty * TX + tx] = sb;
  lds_barrier();
  if (ty == 0 && i < P) {
#pragma unroll
    for (int y = 1; y < TY; ++y) {
      sg += fold_g[y * TX + tx];
      sb += fold_b[y * TX + tx];
    }
    if (dgamma) dgamma[i] = sg + (accum_g ? dgamma[i] : 0.f);
    if (dbeta) dbeta[i] = sb + (accum_b ? dbeta[i] : 0.f);
  }
}

// Per-sample parameters: element-wise.  Either output may be null.
template <int UNUSED = 0>
__global__ void __launch_bounds__(256)
pair_split_kernel(const float *__restrict__ pairs, int total, float *__restrict__ dgamma,
                  float *__restrict__ dbeta, int accum_g, int accum_b) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float2 v = reinterpret_cast<const float2 *>(pairs)[i];
  if (dgamma) dgamma[i] = v.x + (accum_g ? dgamma[i] : 0.f);
  if (dbeta) dbeta[i] = v.y + (accum_b ? dbeta[i] : 0.f);
}

// Launches what (dgamma, dbeta, bc_gamma, bc_beta) ask for; tag names the
// launches for the profiling hooks.
inline int launch_pair_param_reduce(const char *tag, const float *pairs, int64_t batch, int64_t P, float *dgamma,
                                    float *dbeta, int bc_gamma, int bc_beta, int accum_g,
                                    int accum_b, hipStream_t st) {
  float *sum_g = bc_gamma ? dgamma : nullptr, *sum_b = bc_beta ? dbeta : nullptr;
  float *own_g = bc_gamma ? nullptr : dgamma, *own_b = bc_beta ? nullptr : dbeta;
  if (sum_g || sum_b) {
    constexpr int TY = 8;
    NBLAHIP_LAUNCH(tag, pair_batch_sum_kernel<TY>,
                   dim3(static_cast<unsigned>((P + 256 / TY - 1) / (256 / TY))), dim3(256), 0, st,
                   pairs, static_cast<int>(batch), static_cast<int>(P), sum_g, sum_b, accum_g,
                   accum_b);
    if (int e = last_launch_status()) return e;
  }
  if (own_g || own_b) {
    const int64_t total = batch * P;
    NBLAHIP_LAUNCH(tag, pair_split_kernel<0>,
                   dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st, pairs,
                   static_cast<int>(total), own_g, own_b, accum_g, accum_b);
    if (int e = last_launch_status()) return e;
  }
  return 0;
}

} // namespace nblahip
