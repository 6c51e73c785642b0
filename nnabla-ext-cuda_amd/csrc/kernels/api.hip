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

// BatchNormalization tensors of 2^31 elements and more.  A channel runs
// through the whole tensor, so ranges of samples are not independent of each
// other as the rows of the other functions are: they run as the steps of a
// batch that is split over workers - local statistics per range, their merge,
// the normalization per range; backward: the local sums per range, their sum,
// dx per range - with the ranges' statistics and sums behind the launches' own
// workspace.  (The reference indexes these tensors with int and has no such
// path.)  One sample must stay below 2^31 elements.
struct BnRanges {
  int64_t per = 0; // samples (size0 slices) per range
  int count = 0;   // ranges; 0: the tensor fits one launch
};

// 0: proceed (r.count == 0: one launch); 1: empty tensor; <0: error.
int bn_ranges(int64_t size0, int64_t C, int64_t size2, BnRanges &r) {
  const int d = check_dims_units(size0, C, size2);
  if (d) return d;
  r.per = units_per_launch(size0, C * size2);
  r.count = r.per >= size0 ? 0 : static_cast<int>((size0 + r.per - 1) / r.per);
  return 0;
}

size_t bn_stats_floats(int64_t C) { return 2 * static_cast<size_t>(C) + 1; }

// Workspace of a ranged call: [a launch's workspace][statistics count x (2C+1)]
// [pair sums count x 2C][their total 2C], each part 256-byte aligned.
struct BnRangedWs {
  size_t launch = 0, stats = 0, sums = 0, total = 0;
  size_t bytes() const { return launch + stats + sums + total; }
};

BnRangedWs bn_ranged_ws(int64_t size0, int64_t C, int64_t size2, int dtype, const BnRanges &r) {
  auto up = [](size_t b) { return (b + 255) / 256 * 256; };
  BnRangedWs w;
  w.launch = up(chunked_workspace(size0, r.per, [&](int64_t n) { return bn_workspace_bytes(n, C, size2, dtype); }));
  w.stats = up(static_cast<size_t>(r.count) * bn_stats_floats(C) * sizeof(float));
  w.sums = up(static_cast<size_t>(r.count) * 2 * static_cast<size_t>(C) * sizeof(float));
  w.total = up(2 * static_cast<size_t>(C) * sizeof(float));
  return w;
}

size_t bn_any_workspace_bytes(int64_t size0, int64_t C, int64_t size2, int dtype) {
  BnRanges r;
  if (bn_ranges(size0, C, size2, r) != 0) return 0;
  if (r.count == 0) return bn_workspace_bytes(size0, C, size2, dtype);
  return bn_ranged_ws(size0, C, size2, dtype, r).bytes();
}

const void *advance(const void *p, int64_t elems, int dtype) {
  return p ? static_cast<const char *>(p) + static_cast<size_t>(elems) * (dtype == NBLAHIP_F16 ? 2 : 4) : nullptr;
}
void *advance(void *p, int64_t elems, int dtype) {
  return p ? static_cast<char *>(p) + static_cast<size_t>(elems) * (dtype == NBLAHIP_F16 ? 2 : 4) : nullptr;
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
  BnRanges ranges;
  const int d = bn_ranges(size0, size1, size2, ranges);
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
  if (ranges.count == 0) return launch_bn_infer(p, as_stream(stream));
  // (elementwise: the ranges need nothing from each other)
  for (int64_t s0 = 0; s0 < size0; s0 += ranges.per) {
    BnProblem q = p;
    const int64_t at = s0 * size1 * size2;
    q.size0 = std::min(ranges.per, size0 - s0);
    q.x = advance(x, at, dtype);
    q.z = advance(z, at, dtype);
    q.out = advance(y, at, dtype);
    if (int e = launch_bn_infer(q, as_stream(stream))) return e;
  }
  return 0;
}

int bn_fwd_train_impl(const void *x, const void *z, int relu, const float *gamma,
                      const float *beta, void *y, float *batch_mean, float *batch_var,
                      float *rmean, float *rvar, int64_t size0, int64_t size1, int64_t size2,
                      float decay_rate, float eps, int dtype, void *workspace,
                      size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return NBLAHIP_EINVAL;
  BnRanges ranges;
  const int d = bn_ranges(size0, size1, size2, ranges);
  if (d) return d < 0 ? d : 0;
  if (!x || !y || !batch_mean || !batch_var) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(size0) * size1 * size2 * elem_bytes(dtype);
    if (check_in_place(y, x, tb) || check_in_place(y, z, tb)) return NBLAHIP_EALIAS;
  }
  if (int e = check_ws(workspace, workspace_bytes, bn_any_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  if (ranges.count > 0) {
    hipStream_t st = as_stream(stream);
    const BnRangedWs w = bn_ranged_ws(size0, size1, size2, dtype, ranges);
    float *stats = reinterpret_cast<float *>(static_cast<char *>(workspace) + w.launch);
    const size_t stride = bn_stats_floats(size1);
    int i = 0;
    for (int64_t s0 = 0; s0 < size0; s0 += ranges.per, ++i) {
      BnProblem q;
      q.dtype = dtype;
      q.x = advance(x, s0 * size1 * size2, dtype);
      q.batch_mean = stats + i * stride;
      q.batch_var = stats + i * stride + size1;
      q.size0 = std::min(ranges.per, size0 - s0);
      q.C = size1;
      q.size2 = size2;
      q.ws = workspace;
      q.ws_bytes = w.launch;
      if (int e = launch_bn_local_stats(q, st)) return e;
      // (the range's count: its elements per channel, as the merge's weight)
      if (int e = nblahip_fill(stats + i * stride + 2 * size1, NBLAHIP_F32,
                               static_cast<float>(static_cast<double>(q.size0) * static_cast<double>(size2)), 1, st))
        return e;
    }
    if (int e = launch_bn_merge_stats(stats, ranges.count, size1, batch_mean, batch_var, rmean, rvar,
                                      decay_rate, st))
      return e;
    for (int64_t s0 = 0; s0 < size0; s0 += ranges.per) {
      BnProblem q;
      const int64_t at = s0 * size1 * size2;
      q.dtype = dtype;
      q.x = advance(x, at, dtype);
      q.z = advance(z, at, dtype);
      q.out = advance(y, at, dtype);
      q.mean = batch_mean;
      q.var = batch_var;
      q.gamma = gamma;
      q.beta = beta;
      q.size0 = std::min(ranges.per, size0 - s0);
      q.C = size1;
      q.size2 = size2;
      q.eps = eps;
      q.relu = relu;
      if (int e = launch_bn_infer(q, st)) return e;
    }
    return 0;
  }
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
  BnRanges ranges;
  const int d = bn_ranges(size0, size1, size2, ranges);
  if (d) return d < 0 ? d : 0;
  // (the fused backward, which gates dy by the stored output on the way, has no ranged form)
  if (ranges.count > 0 && fused) return NBLAHIP_ERANGE;
  if (!x || !dy || !mean || !var) return NBLAHIP_EINVAL;
  if (fused ? !y_out : (y_out || dz)) return NBLAHIP_EINVAL;
  {
    const size_t tb = static_cast<size_t>(size0) * size1 * size2 * elem_bytes(dtype);
    if (check_in_place(dx, x, tb) || check_in_place(dx, dy, tb) || check_in_place(dz, dy, tb) ||
        ranges_overlap(dz, tb, x, tb))
      return NBLAHIP_EALIAS;
  }
  if (int e = check_ws(workspace, workspace_bytes, bn_any_workspace_bytes(size0, size1, size2, dtype)))
    return e;
  if (ranges.count > 0) {
    hipStream_t st = as_stream(stream);
    const BnRangedWs w = bn_ranged_ws(size0, size1, size2, dtype, ranges);
    float *sums = reinterpret_cast<float *>(static_cast<char *>(workspace) + w.launch + w.stats);
    float *total = reinterpret_cast<float *>(static_cast<char *>(workspace) + w.launch + w.stats + w.sums);
    BnProblem base;
    base.dtype = dtype;
    base.gamma = gamma;
    base.mean = mean;
    base.var = var;
    base.C = size1;
    base.size2 = size2;
    base.eps = eps;
    base.ws = workspace;
    base.ws_bytes = w.launch;
    int i = 0;
    for (int64_t s0 = 0; s0 < size0; s0 += ranges.per, ++i) {
      BnProblem q = base;
      const int64_t at = s0 * size1 * size2;
      q.x = advance(x, at, dtype);
      q.dy = advance(dy, at, dtype);
      q.size0 = std::min(ranges.per, size0 - s0);
      q.dgamma = dgamma;
      q.dbeta = dbeta;
      q.accum_g = i == 0 ? accum_dgamma : 1;
      q.accum_b = i == 0 ? accum_dbeta : 1;
      q.batch_stat = batch_stat;
      if (batch_stat) {
        q.sums_out = sums + static_cast<size_t>(i) * 2 * size1; // this range's (sum dy*(x-mean), sum dy)
      } else {
        q.out = advance(dx, at, dtype); // fixed statistics: dx is elementwise
        q.accum_dx = accum_dx;
      }
      if (int e = launch_bn_bwd(q, st)) return e;
    }
    if (!batch_stat || !dx) return 0;
    if (int e = launch_sum_rows(sums, ranges.count, 2 * size1, total, st)) return e;
    for (int64_t s0 = 0; s0 < size0; s0 += ranges.per) {
      BnProblem q = base;
      const int64_t at = s0 * size1 * size2;
      q.x = advance(x, at, dtype);
      q.dy = advance(dy, at, dtype);
      q.out = advance(dx, at, dtype);
      q.size0 = std::min(ranges.per, size0 - s0);
      q.dmean = dmean;
      q.dvar = dvar;
      q.sums_in = total;
      q.total_count = static_cast<double>(size0) * static_cast<double>(size2);
      q.accum_dx = accum_dx;
      if (int e = launch_bn_bwd_from_sums(q, st)) return e;
    }
    return 0;
  }
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
  if (!dtype_ok(dtype)) return 0;
  return bn_any_workspace_bytes(size0, size1, size2, dtype);
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
