// C-ABI entry points of the normalization kernels: argument validation and
// translation into launch-layer problems.  Nothing here allocates, throws or
// waits for the device.
#include <algorithm>
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

// The kernels index a tensor with 32 bits.  The reduction units of the row
// normalizations are independent of each other - LayerNormalization rows, the
// samples of Group / InstanceNormalization - so a tensor of 2^31 elements and
// more (the reference indexes these with Size_t: layer_normalization.cu:99,
// group_normalization.cu:57-62) runs as several launches over ranges of units,
// each below 2^31 elements; the parameter gradients of the later ranges
// accumulate onto the first range's.  One unit alone must stay below 2^31
// elements.  0: proceed; 1: empty tensor; <0: error.
int check_dims_units(int64_t units, int64_t b, int64_t c) {
  if (units < 0 || b < 0 || c < 0) return NBLAHIP_EINVAL;
  if (units == 0 || b == 0 || c == 0) return 1;
  if (units > kMaxElems || b > kMaxElems || c > kMaxElems) return NBLAHIP_ERANGE;
  if (static_cast<__int128>(b) * c > kMaxElems) return NBLAHIP_ERANGE;
  return 0;
}

// Units per launch: as many as stay below 2^31 elements (and below `cap`).
int64_t units_per_launch(int64_t units, int64_t unit_elems, int64_t cap = kMaxElems) {
  return std::max<int64_t>(1, std::min(units, std::min(cap, kMaxElems / std::max<int64_t>(1, unit_elems))));
}

// Workspace of a call that runs in ranges of `per` units: the larger of what
// a full range and the last, shorter one need.
template <class F> size_t chunked_workspace(int64_t units, int64_t per, F bytes_of) {
  const int64_t tail = units % per;
  return std::max(bytes_of(std::min(units, per)), tail ? bytes_of(tail) : size_t{0});
}

// The range [u0, u0 + n) of the units of a row problem.  unit_rows: statistics
// rows per unit (LayerNormalization: 1; GN: groups; IN: channels).
RowProblem row_range(const RowProblem &p, int64_t u0, int64_t n, int64_t unit_rows, bool is_ln) {
  RowProblem q = p;
  const size_t esz = p.dtype == NBLAHIP_F16 ? 2 : 4;
  const size_t unit_elems = static_cast<size_t>(unit_rows) * static_cast<size_t>(p.R);
  const size_t off = static_cast<size_t>(u0) * unit_elems * esz;
  q.x = static_cast<const char *>(p.x) + off;
  if (p.dy) q.dy = static_cast<const char *>(p.dy) + off;
  if (p.out) q.out = static_cast<char *>(p.out) + off;
  const int64_t r0 = u0 * unit_rows;
  if (p.mean) q.mean = p.mean + r0;
  if (p.var) q.var = p.var + r0;
  if (p.dmean) q.dmean = p.dmean + r0;
  if (p.dvar) q.dvar = p.dvar + r0;
  q.rows = n * unit_rows;
  if (!is_ln) {
    q.batch = n;
    // per-sample InstanceNormalization parameters move with the samples; shared
    // ones accumulate over the ranges
    if (!p.bc_gamma) {
      if (p.gamma) q.gamma = p.gamma + u0 * p.channels;
      if (p.dgamma) q.dgamma = p.dgamma + u0 * p.channels;
    }
    if (!p.bc_beta) {
      if (p.beta) q.beta = p.beta + u0 * p.channels;
      if (p.dbeta) q.dbeta = p.dbeta + u0 * p.channels;
    }
  }
  if (u0 > 0) {
    if (is_ln || p.bc_gamma) q.accum_g = 1;
    if (is_ln || p.bc_beta) q.accum_b = 1;
  }
  return q;
}

int run_rows(const RowProblem &p, int64_t units, int64_t unit_rows, bool is_ln, bool forward,
             hipStream_t st) {
  const int64_t per = units_per_launch(units, unit_rows * p.R);
  if (per >= units) return forward ? launch_row_fwd(p, st) : launch_row_bwd(p, st);
  for (int64_t u0 = 0; u0 < units; u0 += per) {
    const RowProblem q = row_range(p, u0, std::min(per, units - u0), unit_rows, is_ln);
    if (const int e = forward ? launch_row_fwd(q, st) : launch_row_bwd(q, st)) return e;
  }
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
  const int d = check_dims_units(outer, reduce, 1);
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
  return run_rows(p, outer, 1, true, true, as_stream(stream));
}

static size_t ln_bwd_workspace(int64_t outer, int64_t reduce) {
  return chunked_workspace(outer, units_per_launch(outer, reduce),
                           [&](int64_t n) { return row_bwd_workspace_bytes(kRowLN, n, reduce, 0); });
}

size_t nblahip_ln_bwd_workspace_bytes(int64_t outer, int64_t reduce, int dtype) {
  if (!dtype_ok(dtype) || check_dims_units(outer, reduce, 1) != 0) return 0;
  return ln_bwd_workspace(outer, reduce);
}

int nblahip_ln_bwd(const void *x, const void *dy, const float *gamma, const float *mean,
                   const float *var, const float *dmean, const float *dvar, void *dx,
                   float *dgamma, float *dbeta, int accum_dx, int accum_dgamma, int accum_dbeta,
                   int64_t outer, int64_t reduce, float eps, int dtype, void *workspace,
                   size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims_units(outer, reduce, 1);
  if (d) return d < 0 ? d : 0;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (int e = check_ws(workspace, workspace_bytes, ln_bwd_workspace(outer, reduce))) return e;
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
  return run_rows(p, outer, 1, true, false, as_stream(stream));
}

// ----------------------------------------------------------------------------
// GroupNormalization
// ----------------------------------------------------------------------------
static int gn_problem(RowProblem &p, int64_t batch, int64_t channels, int64_t spatial, int groups,
                      int dtype) {
  if (!dtype_ok(dtype) || groups <= 0) return NBLAHIP_EINVAL;
  const int d = check_dims_units(batch, channels, spatial);
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
  return run_rows(p, batch, groups, false, true, as_stream(stream));
}

// (mode kRowGN or kRowIN; unit_rows = statistics rows per sample)
static size_t planes_bwd_workspace(int mode, const RowProblem &p, int64_t unit_rows) {
  return chunked_workspace(p.batch, units_per_launch(p.batch, p.channels * p.spatial), [&](int64_t n) {
    return row_bwd_workspace_bytes(mode, n * unit_rows, p.R, n * p.channels);
  });
}

size_t nblahip_gn_bwd_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial,
                                      int groups, int dtype) {
  RowProblem p;
  if (gn_problem(p, batch, channels, spatial, groups, dtype) != 0) return 0;
  return planes_bwd_workspace(kRowGN, p, groups);
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
  if (int e = check_ws(workspace, workspace_bytes, planes_bwd_workspace(kRowGN, p, groups))) return e;
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
  return run_rows(p, batch, groups, false, false, as_stream(stream));
}

// ----------------------------------------------------------------------------
// InstanceNormalization
// ----------------------------------------------------------------------------
static int in_problem(RowProblem &p, int64_t batch, int64_t channels, int64_t spatial,
                      int bc_gamma, int bc_beta, int dtype) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  const int d = check_dims_units(batch, channels, spatial);
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
  return run_rows(p, batch, channels, false, true, as_stream(stream));
}

size_t nblahip_in_bwd_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial,
                                      int dtype) {
  RowProblem p;
  if (in_problem(p, batch, channels, spatial, 1, 1, dtype) != 0) return 0;
  return planes_bwd_workspace(kRowIN, p, channels);
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
  if (int e = check_ws(workspace, workspace_bytes, planes_bwd_workspace(kRowIN, p, channels))) return e;
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
  return run_rows(p, batch, channels, false, false, as_stream(stream));
}

// ---------------------------------------------------------------------------
// Channel-last Group/InstanceNormalization: x is [batch, spatial, channels].
// ---------------------------------------------------------------------------
namespace {
// 0: run; >0: nothing to do; <0: error.
int cl_problem(ClProblem &p, int64_t batch, int64_t spatial, int64_t channels, int groups,
               int dtype) {
  if (!dtype_ok(dtype) || groups <= 0) return NBLAHIP_EINVAL;
  const int d = check_dims_units(batch, spatial, channels);
  if (d) return d;
  if (channels % groups != 0) return NBLAHIP_EINVAL;
  p.dtype = dtype;
  p.batch = batch;
  p.spatial = spatial;
  p.channels = channels;
  p.groups = groups;
  return 0;
}

// Samples per launch: the kernels put the sample on a grid axis (65535 at
// most) and index a launch's tensor with 32 bits; larger batches and tensors
// run as several launches over ranges of samples (see check_dims_units).
constexpr int64_t kClMaxBatch = 65535;
int64_t cl_per_launch(const ClProblem &p) {
  return units_per_launch(p.batch, p.spatial * p.channels, kClMaxBatch);
}
size_t cl_workspace(const ClProblem &p) {
  return chunked_workspace(p.batch, cl_per_launch(p), [&](int64_t n) {
    return cl_workspace_bytes(n, p.spatial, p.channels, p.dtype);
  });
}
int run_cl(const ClProblem &p, bool forward, hipStream_t st) {
  const int64_t per = cl_per_launch(p);
  if (per >= p.batch) return forward ? launch_cl_fwd(p, st) : launch_cl_bwd(p, st);
  const size_t esz = elem_bytes(p.dtype);
  for (int64_t u0 = 0; u0 < p.batch; u0 += per) {
    ClProblem q = p;
    q.batch = std::min(per, p.batch - u0);
    const size_t off = static_cast<size_t>(u0) * p.spatial * p.channels * esz;
    q.x = static_cast<const char *>(p.x) + off;
    if (p.dy) q.dy = static_cast<const char *>(p.dy) + off;
    if (p.out) q.out = static_cast<char *>(p.out) + off;
    const int64_t r0 = u0 * p.groups;
    q.mean = p.mean + r0;
    q.var = p.var + r0;
    if (p.dmean) q.dmean = p.dmean + r0;
    if (p.dvar) q.dvar = p.dvar + r0;
    if (!p.bc_gamma) {
      if (p.gamma) q.gamma = p.gamma + u0 * p.channels;
      if (p.dgamma) q.dgamma = p.dgamma + u0 * p.channels;
    } else if (u0 > 0) {
      q.accum_g = 1;
    }
    if (!p.bc_beta) {
      if (p.beta) q.beta = p.beta + u0 * p.channels;
      if (p.dbeta) q.dbeta = p.dbeta + u0 * p.channels;
    } else if (u0 > 0) {
      q.accum_b = 1;
    }
    if (const int e = forward ? launch_cl_fwd(q, st) : launch_cl_bwd(q, st)) return e;
  }
  return 0;
}

int cl_fwd(ClProblem &p, const void *x, const float *gamma, const float *beta, void *y,
           float *mean, float *var, float eps, void *workspace, size_t workspace_bytes,
           void *stream) {
  if (!x || !y || !mean || !var) return NBLAHIP_EINVAL;
  if (check_in_place(y, x, static_cast<size_t>(p.batch) * p.spatial * p.channels * elem_bytes(p.dtype)))
    return NBLAHIP_EALIAS;
  if (int e = check_ws(workspace, workspace_bytes, cl_workspace(p))) return e;
  p.x = x;
  p.out = y;
  p.gamma = gamma;
  p.beta = beta;
  p.mean = mean;
  p.var = var;
  p.eps = eps;
  p.ws = workspace;
  p.ws_bytes = workspace_bytes;
  return run_cl(p, true, as_stream(stream));
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
  if (int e = check_ws(workspace, workspace_bytes, cl_workspace(p))) return e;
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
  return run_cl(p, false, as_stream(stream));
}
} // namespace

size_t nblahip_gn_cl_workspace_bytes(int64_t batch, int64_t spatial, int64_t channels, int groups,
                                     int dtype) {
  ClProblem p;
  if (cl_problem(p, batch, spatial, channels, groups, dtype) != 0) return 0;
  return cl_workspace(p);
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
  return cl_workspace(p);
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
