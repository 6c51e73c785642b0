// C-ABI entry points of the normalization kernels: argument validation and
// translation into launch-layer problems.  Nothing here allocates, throws or
// waits for the device.
#include <atomic>

#include "launch.hpp"

using namespace nblahip;

namespace {

constexpr int64_t kMaxElems = (1ll << 31) - 1;

bool dtype_ok(int d) { return d == NBLAHIP_F32 || d == NBLAHIP_F16; }

int check_ws(const void *ws, size_t have, size_t need) {
  if (need == 0) return 0;
  if (!ws || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0 || have < need) return NBLAHIP_EWORKSPACE;
  return 0;
}

// 0: proceed; 1: empty tensor, nothing to do; <0: error.
int check_dims3(int64_t a, int64_t b, int64_t c) {
  if (a < 0 || b < 0 || c < 0) return NBLAHIP_EINVAL;
  if (a == 0 || b == 0 || c == 0) return 1;
  if (a > kMaxElems || b > kMaxElems || c > kMaxElems) return NBLAHIP_ERANGE;
  const __int128 total = static_cast<__int128>(a) * b * c;
  if (total > kMaxElems) return NBLAHIP_ERANGE;
  return 0;
}

hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes) {
  if (!a || !b || !a_bytes || !b_bytes) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

// The row forwards may keep partial statistics in y before they write it, and
// they read gamma/beta while writing y: y may be x itself (in place) but must
// not overlap x partially, nor the parameters, nor the statistics outputs.
int check_fwd_alias(const void *x, void *y, size_t tensor_bytes, const float *gamma, size_t g_bytes,
                    const float *beta, size_t b_bytes, const float *mean, const float *var,
                    size_t stat_bytes) {
  if (y != x && ranges_overlap(x, tensor_bytes, y, tensor_bytes)) return NBLAHIP_EALIAS;
  if (ranges_overlap(y, tensor_bytes, gamma, g_bytes) || ranges_overlap(y, tensor_bytes, beta, b_bytes) ||
      ranges_overlap(y, tensor_bytes, mean, stat_bytes) || ranges_overlap(y, tensor_bytes, var, stat_bytes))
    return NBLAHIP_EALIAS;
  return 0;
}

size_t elem_bytes(int dtype) { return dtype == NBLAHIP_F16 ? 2 : 4; }

// An output tensor may be one of the call's input tensors itself (in place:
// every kernel reads an element before the same thread writes it), but must
// not overlap one in part.
int check_in_place(const void *out, const void *in, size_t tensor_bytes) {
  return out != in && ranges_overlap(out, tensor_bytes, in, tensor_bytes) ? NBLAHIP_EALIAS : 0;
}

// Scratch of nblahip_bn_fwd_train_static, the entry point for callers that
// cannot allocate: one array per GPU in the code object's own data segment,
// held until the process ends.  `scratch` below is only the host-side handle
// of that array; the device address is looked up once per device and kept in
// g_scratch_ptr, and host code passes that pointer, never the handle, to
// kernels.
constexpr size_t kStaticScratchBytes = size_t{4} << 20;
constexpr int kMaxDevices = 64;
__device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of the current device's scratch array (resolved on the first
// call per device; two threads resolving at once store the same address).
int static_scratch(void **out) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return NBLAHIP_EINVAL;
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)); e != hipSuccess)
      return static_cast<int>(e);
    if (!ptr) return static_cast<int>(hipErrorInvalidSymbol);
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return 0;
}

} // namespace

// ----------------------------------------------------------------------------
// BatchNormalization and FusedBatchNormalization (relu != 0: y = max(0, bn + z);
// y_out != null in the backward: dy masked by y_out > 0, masked dy -> dz)
// ----------------------------------------------------------------------------
namespace {
int bn_fwd_infer_impl(const void *x, const void *z, int relu, const float *rmean,
                      const float *rvar, const float *gamma, const float *beta, void *y,
                      int64_t size0, int64_t size1, int64_t size2, float eps, int dtype,
                      void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !rmean || !rvar) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(size0) * size1 * size2 * elem_bytes(dtype);
    if (check_in_place(y, x, tb) || check_in_place(y, z, tb)) return NBLAHIP_EALIAS;
  }
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.out = y;
  p.mean = rmean;
  p.var = rvar;
  p.gamma = gamma;
  p.beta = beta;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.eps = eps;
  p.relu = relu;
  p.z = z;
  return launch_bn_infer(p, as_stream(stream));
}

int bn_fwd_train_impl(const void *x, const void *z, int relu, const float *gamma,
                      const float *beta, void *y, float *batch_mean, float *batch_var,
                      float *rmean, float *rvar, int64_t size0, int64_t size1, int64_t size2,
                      float decay_rate, float eps, int dtype, void *workspace,
                      size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !batch_mean || !batch_var) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(size0) * size1 * size2 * elem_bytes(dtype);
    if (check_in_place(y, x, tb) || check_in_place(y, z, tb)) return NBLAHIP_EALIAS;
  }
  if (int e = check_ws(workspace, workspace_bytes, bn_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.batch_mean = batch_mean;
  p.batch_var = batch_var;
  p.rmean = rmean;
  p.rvar = rvar;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.decay = decay_rate;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  p.relu = relu;
  p.z = z;
  return launch_bn_fwd_train(p, as_stream(stream));
}

int bn_bwd_impl(int fused, const void *x, const void *y_out, const void *dy, const float *gamma,
                const float *mean, const float *var, const float *dmean, const float *dvar,
                void *dx, void *dz, float *dgamma, float *dbeta, int accum_dx, int accum_dz,
                int accum_dgamma, int accum_dbeta, int64_t size0, int64_t size1, int64_t size2,
                float eps, int batch_stat, int dtype, void *workspace, size_t workspace_bytes,
                void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (fused ? !y_out : (y_out || dz)) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(size0) * size1 * size2 * elem_bytes(dtype);
    if (check_in_place(dx, x, tb) || check_in_place(dx, dy, tb) || check_in_place(dz, dy, tb) ||
        ranges_overlap(dz, tb, x, tb))
      return NBLAHIP_EALIAS;
  }
  if (int e = check_ws(workspace, workspace_bytes, bn_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = mean;
  p.var = var;
  p.dmean = batch_stat ? dmean : nullptr;
  p.dvar = batch_stat ? dvar : nullptr;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_dx = accum_dx;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.batch_stat = batch_stat;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  p.y = y_out;
  p.dz = dz;
  p.accum_dz = accum_dz;
  return launch_bn_bwd(p, as_stream(stream));
}
} // namespace

extern "C" {

int nblahip_bn_fwd_infer(const void *x, const float *rmean, const float *rvar,
                         const float *gamma, const float *beta, void *y, int64_t size0,
                         int64_t size1, int64_t size2, float eps, int dtype, void *stream) {
  return bn_fwd_infer_impl(x, nullptr, 0, rmean, rvar, gamma, beta, y, size0, size1, size2, eps,
                           dtype, stream);
}

size_t nblahip_bn_workspace_bytes(int64_t size0, int64_t size1, int64_t size2, int dtype) {
  if (!dtype_ok(dtype) || check_dims3(size0, size1, size2) != 0) return 0;
  return bn_workspace_bytes(size0, size1, size2, dtype);
}

int nblahip_bn_fwd_train(const void *x, const float *gamma, const float *beta, void *y,
                         float *batch_mean, float *batch_var, float *rmean, float *rvar,
                         int64_t size0, int64_t size1, int64_t size2, float decay_rate, float eps,
                         int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return bn_fwd_train_impl(x, nullptr, 0, gamma, beta, y, batch_mean, batch_var, rmean, rvar,
                           size0, size1, size2, decay_rate, eps, dtype, workspace,
                           workspace_bytes, stream);
}

size_t nblahip_bn_fwd_train_static_max_workspace(void) { return kStaticScratchBytes; }

int nblahip_bn_fwd_train_static(const void *x, const float *gamma, const float *beta, void *y,
                                float *batch_mean, float *batch_var, float *rmean, float *rvar,
                                int64_t size0, int64_t size1, int64_t size2, float decay_rate,
                                float eps, int dtype, void *stream) {
  // Shapes whose partials do not fit the static array are turned away before
  // anything touches the device.
  if (dtype_ok(dtype) && check_dims3(size0, size1, size2) == 0 &&
      bn_workspace_bytes(size0, size1, size2, dtype) > kStaticScratchBytes)
    return NBLAHIP_EWORKSPACE;
  void *ws = nullptr;
  if (int e = static_scratch(&ws)) return e;
  // The split reduction writes every partial before it reads it: nothing in
  // the array has to start at zero.
  return bn_fwd_train_impl(x, nullptr, 0, gamma, beta, y, batch_mean, batch_var, rmean, rvar,
                           size0, size1, size2, decay_rate, eps, dtype, ws, kStaticScratchBytes,
                           stream);
}

int nblahip_bn_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                   const float *var, const float *dmean, const float *dvar, void *dx,
                   float *dgamma, float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta,
                   int64_t size0, int64_t size1, int64_t size2, float eps, int batch_stat,
                   int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return bn_bwd_impl(0, x, nullptr, dy, gamma, mean, var, dmean, dvar, dx, nullptr, dgamma, dbeta,
                     accum_dx, 0, accum_dgamma, accum_dbeta, size0, size1, size2, eps, batch_stat,
                     dtype, workspace, workspace_bytes, stream);
}

// ----------------------------------------------------------------------------
// Steps of a BatchNormalization whose batch is split over several workers
// ----------------------------------------------------------------------------
int nblahip_bn_local_stats(const void *x, float *mean, float *var, int64_t size0, int64_t size1,
                           int64_t size2, int dtype, void *workspace, size_t workspace_bytes,
                           void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes, bn_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.batch_mean = mean;
  p.batch_var = var;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_bn_local_stats(p, as_stream(stream));
}

int nblahip_bn_merge_stats(const float *stats, int workers, int64_t channels, float *batch_mean,
                           float *batch_var, float *rmean, float *rvar, float decay_rate,
                           void *stream) {
  if (workers < 0 || channels < 0) return NBLAHIP_EINVAL;
  if (workers == 0 || channels == 0) return 0;
  if (channels > kMaxElems) return NBLAHIP_ERANGE;
  if (!stats || !batch_mean || !batch_var) return NBLAHIP_EINVAL;
  return launch_bn_merge_stats(stats, workers, channels, batch_mean, batch_var, rmean, rvar,
                               decay_rate, as_stream(stream));
}

int nblahip_bn_bwd_local_sums(const void *x, const void *dy, const float *mean, const float *var,
                              float *sums, float *dgamma, float *dbeta, int accum_dgamma,
                              int accum_dbeta, int64_t size0, int64_t size1, int64_t size2,
                              float eps, int dtype, void *workspace, size_t workspace_bytes,
                              void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var || !sums) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes, bn_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.dy = dy;
  p.mean = mean;
  p.var = var;
  p.sums_out = sums;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.batch_stat = 1;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_bn_bwd(p, as_stream(stream));
}

int nblahip_bn_bwd_apply_sums(const void *x, const void *dy, const float *gamma, const float *mean,
                              const float *var, const float *sums, double total_count,
                              const float *dmean, const float *dvar, void *dx, int accum_dx,
                              int64_t size0, int64_t size1, int64_t size2, float eps, int dtype,
                              void *workspace, size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(size0, size1, size2);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var || !sums || !dx || !(total_count >= 1.0)) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes, bn_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  BnProblem p;
  p.dtype = dtype;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = mean;
  p.var = var;
  p.dmean = dmean;
  p.dvar = dvar;
  p.sums_in = sums;
  p.total_count = total_count;
  p.accum_dx = accum_dx;
  p.size0 = size0;
  p.C = size1;
  p.size2 = size2;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_bn_bwd_from_sums(p, as_stream(stream));
}

int nblahip_fused_bn_fwd_infer(const void *x, const void *z, const float *rmean,
                               const float *rvar, const float *gamma, const float *beta, void *y,
                               int64_t size0, int64_t size1, int64_t size2, float eps, int dtype,
                               void *stream) {
  return bn_fwd_infer_impl(x, z, 1, rmean, rvar, gamma, beta, y, size0, size1, size2, eps, dtype,
                           stream);
}

int nblahip_fused_bn_fwd_train(const void *x, const void *z, const float *gamma,
                               const float *beta, void *y, float *batch_mean, float *batch_var,
                               float *rmean, float *rvar, int64_t size0, int64_t size1,
                               int64_t size2, float decay_rate, float eps, int dtype,
                               void *workspace, size_t workspace_bytes, void *stream) {
  return bn_fwd_train_impl(x, z, 1, gamma, beta, y, batch_mean, batch_var, rmean, rvar, size0,
                           size1, size2, decay_rate, eps, dtype, workspace, workspace_bytes,
                           stream);
}

int nblahip_fused_bn_bwd(const void *x, const void *y, const void *dy, const float *gamma,
                         const float *mean, const float *var, const float *dmean,
                         const float *dvar, void *dx, void *dz, float *dgamma, float *dbeta,
                         int accum_dx, int accum_dz, int accum_dgamma, int accum_dbeta,
                         int64_t size0, int64_t size1, int64_t size2, float eps, int batch_stat,
                         int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return bn_bwd_impl(1, x, y, dy, gamma, mean, var, dmean, dvar, dx, dz, dgamma, dbeta, accum_dx,
                     accum_dz, accum_dgamma, accum_dbeta, size0, size1, size2, eps, batch_stat,
                     dtype, workspace, workspace_bytes, stream);
}

// ----------------------------------------------------------------------------
// LayerNormalization
// ----------------------------------------------------------------------------
int nblahip_ln_fwd(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                   float *var, int64_t outer, int64_t reduce, float eps, int dtype,
                   void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(outer, reduce, 1);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_fwd_alias(x, y, static_cast<size_t>(outer) * reduce * elem_bytes(dtype), gamma,
                              reduce * sizeof(float), beta, reduce * sizeof(float), mean, var,
                              outer * sizeof(float)))
    return e;
  RowProblem p;
  p.dtype = dtype;
  p.mode = kRowLN;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.mean = mean;
  p.var = var;
  p.rows = outer;
  p.R = reduce;
  p.eps = eps;
  return launch_row_fwd(p, as_stream(stream));
}

size_t nblahip_ln_bwd_workspace_bytes(int64_t outer, int64_t reduce, int dtype) {
  if (!dtype_ok(dtype) || check_dims3(outer, reduce, 1) != 0) return 0;
  return row_bwd_workspace_bytes(kRowLN, outer, reduce, 0);
}

int nblahip_ln_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                   const float *var, const float *dmean, const float *dvar, void *dx,
                   float *dgamma, float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta,
                   int64_t outer, int64_t reduce, float eps, int dtype, void *workspace,
                   size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(outer, reduce, 1);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes, row_bwd_workspace_bytes(kRowLN, outer, reduce, 0)))
    return e;
  RowProblem p;
  p.dtype = dtype;
  p.mode = kRowLN;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = const_cast<float *>(mean);
  p.var = const_cast<float *>(var);
  p.dmean = dmean;
  p.dvar = dvar;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_dx = accum_dx;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.rows = outer;
  p.R = reduce;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_row_bwd(p, as_stream(stream));
}

// ----------------------------------------------------------------------------
// GroupNormalization
// ----------------------------------------------------------------------------
static int gn_problem(RowProblem &p, int64_t batch, int64_t channels, int64_t spatial, int groups,
                      int dtype) {
  if (!dtype_ok(dtype) || groups <= 0) return NBLAHIP_EINVAL;
  const int d = check_dims3(batch, channels, spatial);
  if (d) return d;
  if (channels % groups != 0) return NBLAHIP_EINVAL;
  p.dtype = dtype;
  p.mode = kRowGN;
  p.batch = batch;
  p.channels = channels;
  p.spatial = spatial;
  p.groups = groups;
  p.rows = batch * groups;
  p.R = (channels / groups) * spatial;
  return 0;
}

int nblahip_gn_fwd(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                   float *var, int64_t batch, int64_t channels, int64_t spatial, int groups,
                   float eps, int dtype, void *stream) {
  RowProblem p;
  const int d = gn_problem(p, batch, channels, spatial, groups, dtype);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_fwd_alias(x, y, static_cast<size_t>(batch) * channels * spatial * elem_bytes(dtype),
                              gamma, channels * sizeof(float), beta, channels * sizeof(float), mean,
                              var, static_cast<size_t>(batch) * groups * sizeof(float)))
    return e;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.mean = mean;
  p.var = var;
  p.eps = eps;
  return launch_row_fwd(p, as_stream(stream));
}

size_t nblahip_gn_bwd_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial,
                                      int groups, int dtype) {
  RowProblem p;
  if (gn_problem(p, batch, channels, spatial, groups, dtype) != 0) return 0;
  return row_bwd_workspace_bytes(kRowGN, p.rows, p.R, batch * channels);
}

int nblahip_gn_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                   const float *var, const float *dmean, const float *dvar, void *dx,
                   float *dgamma, float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta,
                   int64_t batch, int64_t channels, int64_t spatial, int groups, float eps,
                   int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  RowProblem p;
  const int d = gn_problem(p, batch, channels, spatial, groups, dtype);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes,
                       row_bwd_workspace_bytes(kRowGN, p.rows, p.R, batch * channels)))
    return e;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = const_cast<float *>(mean);
  p.var = const_cast<float *>(var);
  p.dmean = dmean;
  p.dvar = dvar;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_dx = accum_dx;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_row_bwd(p, as_stream(stream));
}

// ----------------------------------------------------------------------------
// InstanceNormalization
// ----------------------------------------------------------------------------
static int in_problem(RowProblem &p, int64_t batch, int64_t channels, int64_t spatial,
                      int bc_gamma, int bc_beta, int dtype) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims3(batch, channels, spatial);
  if (d) return d;
  p.dtype = dtype;
  p.mode = kRowIN;
  p.batch = batch;
  p.channels = channels;
  p.spatial = spatial;
  p.groups = static_cast<int>(channels);
  p.bc_gamma = bc_gamma != 0;
  p.bc_beta = bc_beta != 0;
  p.rows = batch * channels;
  p.R = spatial;
  return 0;
}

int nblahip_in_fwd(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                   float *var, int64_t batch, int64_t channels, int64_t spatial, int bc_gamma,
                   int bc_beta, float eps, int dtype, void *stream) {
  RowProblem p;
  const int d = in_problem(p, batch, channels, spatial, bc_gamma, bc_beta, dtype);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_fwd_alias(x, y, static_cast<size_t>(batch) * channels * spatial * elem_bytes(dtype),
                              gamma, (bc_gamma ? 1 : batch) * channels * sizeof(float), beta,
                              (bc_beta ? 1 : batch) * channels * sizeof(float), mean, var,
                              static_cast<size_t>(batch) * channels * sizeof(float)))
    return e;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.mean = mean;
  p.var = var;
  p.eps = eps;
  return launch_row_fwd(p, as_stream(stream));
}

size_t nblahip_in_bwd_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial,
                                      int dtype) {
  RowProblem p;
  if (in_problem(p, batch, channels, spatial, 1, 1, dtype) != 0) return 0;
  return row_bwd_workspace_bytes(kRowIN, p.rows, p.R, batch * channels);
}

int nblahip_in_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                   const float *var, const float *dmean, const float *dvar, void *dx,
                   float *dgamma, float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta,
                   int64_t batch, int64_t channels, int64_t spatial, int bc_gamma, int bc_beta,
                   float eps, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  RowProblem p;
  const int d = in_problem(p, batch, channels, spatial, bc_gamma, bc_beta, dtype);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes,
                       row_bwd_workspace_bytes(kRowIN, p.rows, p.R, batch * channels)))
    return e;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = const_cast<float *>(mean);
  p.var = const_cast<float *>(var);
  p.dmean = dmean;
  p.dvar = dvar;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_dx = accum_dx;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_row_bwd(p, as_stream(stream));
}

// ---------------------------------------------------------------------------
// Channel-last Group/InstanceNormalization: x is [batch, spatial, channels].
// ---------------------------------------------------------------------------
namespace {
// 0: run; >0: nothing to do; <0: error.
int cl_problem(ClProblem &p, int64_t batch, int64_t spatial, int64_t channels, int groups,
               int dtype) {
  if (!dtype_ok(dtype) || groups <= 0) return NBLAHIP_EINVAL;
  const int d = check_dims3(batch, spatial, channels);
  if (d) return d;
  if (channels % groups != 0) return NBLAHIP_EINVAL;
  if (batch > 65535) return NBLAHIP_ERANGE; // one slab per grid y/z index
  p.dtype = dtype;
  p.batch = batch;
  p.spatial = spatial;
  p.channels = channels;
  p.groups = groups;
  return 0;
}

int cl_fwd(ClProblem &p, const void *x, const float *gamma, const float *beta, void *y,
           float *mean, float *var, float eps, void *workspace, size_t workspace_bytes,
           void *stream) {
  if (!x || !y || !mean || !var) return NBLAHIP_EINVAL;
  if (check_in_place(y, x, static_cast<size_t>(p.batch) * p.spatial * p.channels * elem_bytes(p.dtype)))
    return NBLAHIP_EALIAS;
  if (int e = check_ws(workspace, workspace_bytes,
                       cl_workspace_bytes(p.batch, p.spatial, p.channels, p.dtype)))
    return e;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.mean = mean;
  p.var = var;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_cl_fwd(p, as_stream(stream));
}

int cl_bwd(ClProblem &p, const void *x, const void *dy, const float *gamma, const float *mean,
           const float *var, const float *dmean, const float *dvar, void *dx, float *dgamma,
           float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta, float eps,
           void *workspace, size_t workspace_bytes, void *stream) {
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(p.batch) * p.spatial * p.channels * elem_bytes(p.dtype);
    if (check_in_place(dx, x, tb) || check_in_place(dx, dy, tb)) return NBLAHIP_EALIAS;
  }
  if (int e = check_ws(workspace, workspace_bytes,
                       cl_workspace_bytes(p.batch, p.spatial, p.channels, p.dtype)))
    return e;
  p.x = x;
  p.dy = dy;
  p.out = dx;
  p.gamma = gamma;
  p.mean = const_cast<float *>(mean);
  p.var = const_cast<float *>(var);
  p.dmean = dmean;
  p.dvar = dvar;
  p.dgamma = dgamma;
  p.dbeta = dbeta;
  p.accum_dx = accum_dx;
  p.accum_g = accum_dgamma;
  p.accum_b = accum_dbeta;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return launch_cl_bwd(p, as_stream(stream));
}
} // namespace

size_t nblahip_gn_cl_workspace_bytes(int64_t batch, int64_t spatial, int64_t channels, int groups,
                                     int dtype) {
  ClProblem p;
  if (cl_problem(p, batch, spatial, channels, groups, dtype) != 0) return 0;
  return cl_workspace_bytes(batch, spatial, channels, dtype);
}

int nblahip_gn_cl_fwd(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                      float *var, int64_t batch, int64_t spatial, int64_t channels, int groups,
                      float eps, int dtype, void *workspace, size_t workspace_bytes,
                      void *stream) {
  ClProblem p;
  const int d = cl_problem(p, batch, spatial, channels, groups, dtype);
  if (d) return d < 0 ? d : 0;
  return cl_fwd(p, x, gamma, beta, y, mean, var, eps, workspace, workspace_bytes, stream);
}

int nblahip_gn_cl_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                      const float *var, const float *dmean, const float *dvar, void *dx,
                      float *dgamma, float *dbeta, int accum_dx, int accum_dgamma,
                      int accum_dbeta, int64_t batch, int64_t spatial, int64_t channels,
                      int groups, float eps, int dtype, void *workspace, size_t workspace_bytes,
                      void *stream) {
  ClProblem p;
  const int d = cl_problem(p, batch, spatial, channels, groups, dtype);
  if (d) return d < 0 ? d : 0;
  return cl_bwd(p, x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta, accum_dx,
                accum_dgamma, accum_dbeta, eps, workspace, workspace_bytes, stream);
}

size_t nblahip_in_cl_workspace_bytes(int64_t batch, int64_t spatial, int64_t channels,
                                     int dtype) {
  ClProblem p;
  if (cl_problem(p, batch, spatial, channels, static_cast<int>(std::max<int64_t>(channels, 1)),
                 dtype) != 0)
    return 0;
  return cl_workspace_bytes(batch, spatial, channels, dtype);
}

int nblahip_in_cl_fwd(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                      float *var, int64_t batch, int64_t spatial, int64_t channels, int bc_gamma,
                      int bc_beta, float eps, int dtype, void *workspace, size_t workspace_bytes,
                      void *stream) {
  ClProblem p;
  const int d = cl_problem(p, batch, spatial, channels,
                           static_cast<int>(std::max<int64_t>(channels, 1)), dtype);
  if (d) return d < 0 ? d : 0;
  p.bc_gamma = bc_gamma;
  p.bc_beta = bc_beta;
  return cl_fwd(p, x, gamma, beta, y, mean, var, eps, workspace, workspace_bytes, stream);
}

int nblahip_in_cl_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                      const float *var, const float *dmean, const float *dvar, void *dx,
                      float *dgamma, float *dbeta, int accum_dx, int accum_dgamma,
                      int accum_dbeta, int64_t batch, int64_t spatial, int64_t channels,
                      int bc_gamma, int bc_beta, float eps, int dtype, void *workspace,
                      size_t workspace_bytes, void *stream) {
  ClProblem p;
  const int d = cl_problem(p, batch, spatial, channels,
                           static_cast<int>(std::max<int64_t>(channels, 1)), dtype);
  if (d) return d < 0 ? d : 0;
  p.bc_gamma = bc_gamma;
  p.bc_beta = bc_beta;
  return cl_bwd(p, x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta, accum_dx,
                accum_dgamma, accum_dbeta, eps, workspace, workspace_bytes, stream);
}

} // extern "C"
