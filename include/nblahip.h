/*
 * nblahip.h - C-ABI of the MI355X (gfx950) normalization kernel layer.
 *
 * This is the whole device-facing surface of the backend: plain pointers and
 * sizes, no C++ types, no exceptions.  The nbla::Function subclasses of the
 * "hip" backend (BatchNormalizationHip<T>, LayerNormalizationHip<T>,
 * GroupNormalizationHip<T>, InstanceNormalizationHip<T>) call nothing else.
 * Each entry point replaces the kernel launches of one reference function
 * body; the citation names that body under sony/nnabla-ext-cuda.
 *
 * Conventions (all entry points):
 *   - return 0 on success, a negative NBLAHIP_E* code for a bad argument, or a
 *     positive hipError_t value for a runtime failure; never throw, never
 *     allocate, never synchronise the host; nblahip_error_string() explains;
 *   - every pointer is a borrowed device pointer on the current device;
 *   - `dtype` is the storage type of the activation tensors x, y, dy, dx
 *     (NBLAHIP_F32 or NBLAHIP_F16).  gamma, beta, their gradients, running
 *     and batch statistics and the statistic gradients are ALWAYS float32,
 *     all arithmetic and accumulation is float32;
 *   - a NULL gamma / beta means no_scale / no_bias (1 and 0); a NULL
 *     dx / dgamma / dbeta means "not propagated"; NULL dmean / dvar means the
 *     function had a single output; `accum_*` != 0 adds onto the existing
 *     gradient instead of overwriting it;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     null stream the reference launches on);
 *   - `workspace` is caller-owned scratch of at least the matching
 *     *_workspace_bytes() (256-byte aligned); its contents need not persist
 *     between calls.  Results are deterministic (no atomics): same inputs,
 *     same bits.
 */
#ifndef NBLAHIP_H_
#define NBLAHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NBLAHIP_EXPORT __attribute__((visibility("default")))

enum nblahip_dtype { NBLAHIP_F32 = 0, NBLAHIP_F16 = 1 };

enum nblahip_status {
  NBLAHIP_OK = 0,
  NBLAHIP_EINVAL = -1,    /* NULL required pointer, non-positive size, bad enum */
  NBLAHIP_EWORKSPACE = -2,/* workspace NULL, misaligned or too small */
  NBLAHIP_ERANGE = -3,    /* 2^31 or more elements in one row / sample / slice ahead of
                             the channel axis, or in a tensor given to an entry point
                             that does not run in ranges */
  NBLAHIP_EALIAS = -4     /* output overlaps an input it must not overlap */
};

/* Human-readable text for a status (negative) or hipError_t (positive). */
NBLAHIP_EXPORT const char *nblahip_error_string(int code);
/* ABI version: bumps when a signature changes. */
NBLAHIP_EXPORT int nblahip_abi_version(void);

/* ------------------------------------------------------------------------
 * BatchNormalization.  x is viewed as [size0, size1, size2] with size1 = C the
 * normalised axis (src/nbla/cuda/function/generic/batch_normalization.cu:34-35,
 * 53-55); size2 == 1 is the channel-last layout.  N = size0*size2.
 *
 * Aliasing: y may be x itself (in place), dx may be x or dy itself; an output
 * that overlaps an input tensor only in part is rejected with NBLAHIP_EALIAS
 * before anything is launched.  In-place calls never take the kernels whose
 * blocks exchange partial sums (a block that gives up waiting for a partner
 * reads the partner's part of the inputs again, which the partner would
 * already be overwriting): they run on the plans without an exchange, with
 * the same results within the summation order.
 *
 * Sizes: a tensor of fewer than 2^31 elements is one sequence of launches.
 * Larger ones run in ranges along size0 - a channel runs through the whole
 * tensor, so the ranges are the steps of a split batch (further down): local
 * statistics per range, nblahip_bn_merge_stats, the normalization per range;
 * backward: the local sums per range, their sum, dx per range.  size1*size2
 * must stay below 2^31; the fused backward has no ranged form.  The reference
 * indexes with int (kernel/batch_normalization.cuh:246-254) and has no such
 * path.
 * ---------------------------------------------------------------------- */

/* Replaces forward_impl_global + forward_global_kernel
 * (batch_normalization.cu:175-199, kernel/batch_normalization.cuh:332-349):
 *   y = (x - rm[c]) * gamma[c] / sqrt(rv[c] + eps) + beta[c]. */
NBLAHIP_EXPORT int nblahip_bn_fwd_infer(const void *x, const float *rmean,
                                        const float *rvar, const float *gamma,
                                        const float *beta, void *y,
                                        int64_t size0, int64_t size1,
                                        int64_t size2, float eps, int dtype,
                                        void *stream);

NBLAHIP_EXPORT size_t nblahip_bn_workspace_bytes(int64_t size0, int64_t size1,
                                                 int64_t size2, int dtype);

/* Replaces forward_impl_batch -> forward_batch_parallel_reduction
 * (batch_normalization.cu:109-172, generic/kernel/batch_normalization.cu:64-111,
 * kernels cuh:259-325) and the cuDNN ForwardTraining(Ex) call of the cudnn
 * context (cudnn/function/generic/batch_normalization.cu:171-261):
 *   batch_mean[c], batch_var[c] (biased) are always written (they are the
 *   saved statistics backward needs);
 *   rmean <- d*rmean + (1-d)*mean, rvar <- d*rvar + (1-d)*var*N/(N-1) when the
 *   pointers are non-NULL (NULL = recompute_impl, no running-stat update);
 *   y = (x-mean)*gamma/sqrt(var+eps)+beta. */
NBLAHIP_EXPORT int nblahip_bn_fwd_train(const void *x, const float *gamma,
                                        const float *beta, void *y,
                                        float *batch_mean, float *batch_var,
                                        float *rmean, float *rvar,
                                        int64_t size0, int64_t size1,
                                        int64_t size2, float decay_rate,
                                        float eps, int dtype, void *workspace,
                                        size_t workspace_bytes, void *stream);

/* nblahip_bn_fwd_train for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as nblahip_bn_fwd_train minus the workspace: the partials of the
 * split reduction live in an array of
 * nblahip_bn_fwd_train_static_max_workspace() bytes (4 MiB) inside the
 * library's code object, one per GPU, held until the process ends.  A shape
 * whose nblahip_bn_workspace_bytes() exceeds that returns NBLAHIP_EWORKSPACE.
 * The call allocates and frees nothing.  All calls on one GPU share the array:
 * calls that overlap in time on the same GPU (different streams or threads)
 * race, so keep them on one stream.  The array's address is looked up on the
 * first call per device; a call with an empty tensor (size0 == 0) does that
 * look-up and launches nothing, which is the set-up step to make before a
 * capture starts. */
NBLAHIP_EXPORT size_t nblahip_bn_fwd_train_static_max_workspace(void);
NBLAHIP_EXPORT int nblahip_bn_fwd_train_static(
    const void *x, const float *gamma, const float *beta, void *y,
    float *batch_mean, float *batch_var, float *rmean, float *rvar,
    int64_t size0, int64_t size1, int64_t size2, float decay_rate, float eps,
    int dtype, void *stream);

/* Replaces backward_impl_batch (batch_normalization.cu:215-316, kernels
 * cuh:402-540) and cudnnBatchNormalizationBackward(Ex)
 * (cudnn/.../batch_normalization.cu:328-457).  mean/var are the statistics the
 * forward used: the batch statistics when batch_stat != 0, the running ones
 * otherwise (inference-mode backward: statistics are constants, so
 * dx = dy*gamma/sqrt(var+eps)).  dmean/dvar (3-output form) only apply to
 * batch_stat != 0. */
NBLAHIP_EXPORT int nblahip_bn_bwd(const void *x, const void *dy,
                                  const float *gamma, const float *mean,
                                  const float *var, const float *dmean,
                                  const float *dvar, void *dx, float *dgamma,
                                  float *dbeta, int accum_dx, int accum_dgamma,
                                  int accum_dbeta, int64_t size0, int64_t size1,
                                  int64_t size2, float eps, int batch_stat,
                                  int dtype, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * BatchNormalization of a batch that is split over several workers
 * (SyncBatchNormalization): the device steps of one worker.  The exchange
 * between the steps (all-gather of the statistics, all-reduce of the backward
 * pairs) belongs to the caller's communicator; with one worker the sequence
 * equals nblahip_bn_fwd_train / nblahip_bn_bwd.
 *   forward : local_stats -> [all-gather stats] -> merge_stats ->
 *             nblahip_bn_fwd_infer(x, batch_mean, batch_var, gamma, beta, y)
 *   backward: bwd_local_sums -> [all-reduce sums] -> bwd_apply_sums
 * ---------------------------------------------------------------------- */

/* Replaces forward_collect_statistics(_channels_last)
 * (sync_batch_normalization.cu:122-131): mean[C] and biased var[C] of this
 * worker's shard.  (The reference exchanges 1/sqrt(var+eps); the variance
 * itself loses nothing when eps dominates it.) */
NBLAHIP_EXPORT int nblahip_bn_local_stats(const void *x, float *mean,
                                          float *var, int64_t size0,
                                          int64_t size1, int64_t size2,
                                          int dtype, void *workspace,
                                          size_t workspace_bytes, void *stream);

/* Replaces forward_reduce_statistics (sync_batch_normalization.cu:146-150,
 * kernel/sync_batch_normalization.cuh:448-487).  stats: `workers` records of
 * 2*channels+1 floats {mean[C], var[C], count}, as gathered.  Writes the
 * statistics of the whole batch and updates the running ones (NULL: not). */
NBLAHIP_EXPORT int nblahip_bn_merge_stats(const float *stats, int workers,
                                          int64_t channels, float *batch_mean,
                                          float *batch_var, float *rmean,
                                          float *rvar, float decay_rate,
                                          void *stream);

/* Replaces backward_reduce(_channels_last) (sync_batch_normalization.cu:
 * 216-231).  mean/var: statistics of the whole batch.  sums[C][2] =
 * (sum dy*(x-mean), sum dy) over this worker's shard, to be summed over the
 * workers; dgamma/dbeta (optional) are this worker's contributions. */
NBLAHIP_EXPORT int nblahip_bn_bwd_local_sums(
    const void *x, const void *dy, const float *mean, const float *var,
    float *sums, float *dgamma, float *dbeta, int accum_dgamma, int accum_dbeta,
    int64_t size0, int64_t size1, int64_t size2, float eps, int dtype,
    void *workspace, size_t workspace_bytes, void *stream);

/* Replaces backward_dx_post(_channels_last) (sync_batch_normalization.cu:
 * 258-283, kernel/sync_batch_normalization.cuh:899-960).  sums: the pairs
 * summed over all workers; total_count: elements per channel over all
 * workers. */
NBLAHIP_EXPORT int nblahip_bn_bwd_apply_sums(
    const void *x, const void *dy, const float *gamma, const float *mean,
    const float *var, const float *sums, double total_count,
    const float *dmean, const float *dvar, void *dx, int accum_dx,
    int64_t size0, int64_t size1, int64_t size2, float eps, int dtype,
    void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * FusedBatchNormalization: y = max(0, BatchNormalization(x) + z), z optional
 * (NULL: no residual input).  Same tensor view, statistics and workspace as
 * BatchNormalization above; gamma and beta are always present in the
 * reference (fused_batch_normalization.hpp:30-37) but may be NULL here.
 * ---------------------------------------------------------------------- */

/* Replaces the batch_stat == false forward of the composite
 * FusedBatchNormalization (BatchNormalization forward_impl_global,
 * batch_normalization.cu:175-199, then add2 and relu,
 * include/nbla/cuda/utils/add2.cuh:23-27, relu.cuh:48-52). */
NBLAHIP_EXPORT int nblahip_fused_bn_fwd_infer(const void *x, const void *z,
                                              const float *rmean,
                                              const float *rvar,
                                              const float *gamma,
                                              const float *beta, void *y,
                                              int64_t size0, int64_t size1,
                                              int64_t size2, float eps,
                                              int dtype, void *stream);

/* Replaces fused_batch_norm_forward: cudnnBatchNormalizationForwardTrainingEx
 * with BN_ADD_ACTIVATION / BN_ACTIVATION
 * (cudnn/function/generic/fused_batch_normalization.cu:136-216). */
NBLAHIP_EXPORT int nblahip_fused_bn_fwd_train(
    const void *x, const void *z, const float *gamma, const float *beta,
    void *y, float *batch_mean, float *batch_var, float *rmean, float *rvar,
    int64_t size0, int64_t size1, int64_t size2, float decay_rate, float eps,
    int dtype, void *workspace, size_t workspace_bytes, void *stream);

/* Replaces cudnnBatchNormalizationBackwardEx
 * (cudnn/function/generic/fused_batch_normalization.cu:230-357) and the
 * composite relu_add2_backward (function/generic/fused_batch_normalization.cu
 * :47-75) followed by the BatchNormalization backward: with
 * g = dy where y > 0 else 0,  dz (+)= g  and (dx, dgamma, dbeta) are the
 * BatchNormalization backward of g.  y is the forward output (required);
 * dx, dz, dgamma, dbeta may each be NULL (not propagated); dz may alias dy. */
NBLAHIP_EXPORT int nblahip_fused_bn_bwd(
    const void *x, const void *y, const void *dy, const float *gamma,
    const float *mean, const float *var, const float *dmean, const float *dvar,
    void *dx, void *dz, float *dgamma, float *dbeta, int accum_dx, int accum_dz,
    int accum_dgamma, int accum_dbeta, int64_t size0, int64_t size1,
    int64_t size2, float eps, int batch_stat, int dtype, void *workspace,
    size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * LayerNormalization.  x viewed as [outer, reduce]
 * (src/nbla/cuda/function/generic/layer_normalization.cu:53-59).
 *
 * The forward entry points of the three row normalizations below take no
 * workspace.  For tensors of a few very long rows they keep partial statistics
 * in the first bytes of y until the pass that writes y overwrites them: y must
 * not overlap x other than being x itself (in place, y == x, is detected and
 * handled without the scratch use), nor gamma, beta, mean or var.  A y that
 * does is rejected with NBLAHIP_EALIAS before anything is launched.
 * ---------------------------------------------------------------------- */

/* Replaces forward_impl (layer_normalization.cu:77-133): reduce_2d_x<WelfordOp>
 * + layer_norm_forward_normalization.  mean[outer], var[outer] (biased) are
 * always written. gamma/beta have `reduce` elements. */
NBLAHIP_EXPORT int nblahip_ln_fwd(const void *x, const float *gamma,
                                  const float *beta, void *y, float *mean,
                                  float *var, int64_t outer, int64_t reduce,
                                  float eps, int dtype, void *stream);

NBLAHIP_EXPORT size_t nblahip_ln_bwd_workspace_bytes(int64_t outer,
                                                     int64_t reduce, int dtype);

/* Replaces backward_impl (layer_normalization.cu:136-279): the four launches
 * reduce_2d_x<LNGradOp>, ..._dx_factor, ..._dx, ..._dbeta_dgamma. */
NBLAHIP_EXPORT int nblahip_ln_bwd(const void *x, const void *dy,
                                  const float *gamma, const float *mean,
                                  const float *var, const float *dmean,
                                  const float *dvar, void *dx, float *dgamma,
                                  float *dbeta, int accum_dx, int accum_dgamma,
                                  int accum_dbeta, int64_t outer,
                                  int64_t reduce, float eps, int dtype,
                                  void *workspace, size_t workspace_bytes,
                                  void *stream);

/* ------------------------------------------------------------------------
 * GroupNormalization.  x viewed as [batch, channels, spatial] (channel-first),
 * statistics per (n, group) over (channels/groups)*spatial elements
 * (src/nbla/cuda/function/generic/group_normalization.cu:57-62).  gamma/beta
 * have `channels` elements.
 * ---------------------------------------------------------------------- */

/* Replaces forward_channel_first (group_normalization.cu:112-186): Welford,
 * normalization_factor and normalization launches.  mean/var: [batch*groups]. */
NBLAHIP_EXPORT int nblahip_gn_fwd(const void *x, const float *gamma,
                                  const float *beta, void *y, float *mean,
                                  float *var, int64_t batch, int64_t channels,
                                  int64_t spatial, int groups, float eps,
                                  int dtype, void *stream);

NBLAHIP_EXPORT size_t nblahip_gn_bwd_workspace_bytes(int64_t batch,
                                                     int64_t channels,
                                                     int64_t spatial,
                                                     int groups, int dtype);

/* Replaces backward_channel_first (group_normalization.cu:227-398): the five
 * launches GNGradOp reduce, gamma_invstd, dx_factor, dx, dbeta_dgamma. */
NBLAHIP_EXPORT int nblahip_gn_bwd(const void *x, const void *dy,
                                  const float *gamma, const float *mean,
                                  const float *var, const float *dmean,
                                  const float *dvar, void *dx, float *dgamma,
                                  float *dbeta, int accum_dx, int accum_dgamma,
                                  int accum_dbeta, int64_t batch,
                                  int64_t channels, int64_t spatial, int groups,
                                  float eps, int dtype, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * InstanceNormalization.  x viewed as [batch, channels, spatial]; statistics
 * per (n, c) (src/nbla/cuda/function/generic/instance_normalization.cu:53-55).
 * bc_gamma / bc_beta != 0: the parameter has `channels` elements and is
 * broadcast over the batch (index row % channels); == 0: it has
 * batch*channels elements (index row)
 * (kernel/instance_normalization.cuh:37-38).
 * ---------------------------------------------------------------------- */

/* Replaces forward_channel_first (instance_normalization.cu:99-174). */
NBLAHIP_EXPORT int nblahip_in_fwd(const void *x, const float *gamma,
                                  const float *beta, void *y, float *mean,
                                  float *var, int64_t batch, int64_t channels,
                                  int64_t spatial, int bc_gamma, int bc_beta,
                                  float eps, int dtype, void *stream);

NBLAHIP_EXPORT size_t nblahip_in_bwd_workspace_bytes(int64_t batch,
                                                     int64_t channels,
                                                     int64_t spatial,
                                                     int dtype);

/* Replaces backward_channel_first (instance_normalization.cu:203-465) including
 * the broadcast-backward sum over the batch (device_sum, :427-464). */
NBLAHIP_EXPORT int nblahip_in_bwd(const void *x, const void *dy,
                                  const float *gamma, const float *mean,
                                  const float *var, const float *dmean,
                                  const float *dvar, void *dx, float *dgamma,
                                  float *dbeta, int accum_dx, int accum_dgamma,
                                  int accum_dbeta, int64_t batch,
                                  int64_t channels, int64_t spatial,
                                  int bc_gamma, int bc_beta, float eps,
                                  int dtype, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Channel-last Group/InstanceNormalization.  x viewed as
 * [batch, spatial, channels] (channel axis last).  The reference transposes
 * to channel-first through ChannelFirstAdaptor before and after its kernels
 * (group_normalization.cu:39-55, :93-106, :203-224;
 * instance_normalization.cu:40-51, :81-94, :187-207); these entry points read
 * and write the channel-last tensor in place of those transposes.  Results
 * equal the channel-first entry points applied to the transposed tensor.
 * Both directions need a workspace of *_cl_workspace_bytes.  Batches beyond
 * 65535 and tensors of 2^31 elements and more run as several launches over
 * ranges of samples (one sample must stay below 2^31 elements).
 * Aliasing as for BatchNormalization: y == x, dx == x and dx == dy are in-place
 * calls and run on the kernels without an exchange between blocks; a partial
 * overlap is rejected with NBLAHIP_EALIAS.
 * ---------------------------------------------------------------------- */
NBLAHIP_EXPORT size_t nblahip_gn_cl_workspace_bytes(int64_t batch,
                                                    int64_t spatial,
                                                    int64_t channels,
                                                    int groups, int dtype);

/* Replaces convert_to_channel_first + forward_channel_first +
 * convert_from_channel_first (group_normalization.cu:93-106). */
NBLAHIP_EXPORT int nblahip_gn_cl_fwd(const void *x, const float *gamma,
                                     const float *beta, void *y, float *mean,
                                     float *var, int64_t batch, int64_t spatial,
                                     int64_t channels, int groups, float eps,
                                     int dtype, void *workspace,
                                     size_t workspace_bytes, void *stream);

/* Replaces the adaptor backward + backward_channel_first
 * (group_normalization.cu:203-224). */
NBLAHIP_EXPORT int nblahip_gn_cl_bwd(const void *x, const void *dy,
                                     const float *gamma, const float *mean,
                                     const float *var, const float *dmean,
                                     const float *dvar, void *dx, float *dgamma,
                                     float *dbeta, int accum_dx,
                                     int accum_dgamma, int accum_dbeta,
                                     int64_t batch, int64_t spatial,
                                     int64_t channels, int groups, float eps,
                                     int dtype, void *workspace,
                                     size_t workspace_bytes, void *stream);

NBLAHIP_EXPORT size_t nblahip_in_cl_workspace_bytes(int64_t batch,
                                                    int64_t spatial,
                                                    int64_t channels,
                                                    int dtype);

/* Replaces convert_to_channel_first + forward_channel_first +
 * convert_from_channel_first (instance_normalization.cu:81-94). */
NBLAHIP_EXPORT int nblahip_in_cl_fwd(const void *x, const float *gamma,
                                     const float *beta, void *y, float *mean,
                                     float *var, int64_t batch, int64_t spatial,
                                     int64_t channels, int bc_gamma, int bc_beta,
                                     float eps, int dtype, void *workspace,
                                     size_t workspace_bytes, void *stream);

/* Replaces the adaptor backward + backward_channel_first
 * (instance_normalization.cu:187-207). */
NBLAHIP_EXPORT int nblahip_in_cl_bwd(const void *x, const void *dy,
                                     const float *gamma, const float *mean,
                                     const float *var, const float *dmean,
                                     const float *dvar, void *dx, float *dgamma,
                                     float *dbeta, int accum_dx,
                                     int accum_dgamma, int accum_dbeta,
                                     int64_t batch, int64_t spatial,
                                     int64_t channels, int bc_gamma, int bc_beta,
                                     float eps, int dtype, void *workspace,
                                     size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Runtime shims used by the backend's array class and singleton so that host
 * C++ never includes a HIP header.  They replace the cudaMalloc / cudaMemcpy /
 * cudaMemset / dtype-converting copy paths of src/nbla/cuda/memory/
 * cuda_memory.cpp:51-75 and src/nbla/cuda/array/cuda_array.cpp:211-347, and
 * cuda_set_device / device synchronisation of src/nbla/cuda/common.cpp:20-32,
 * src/nbla/cuda/cuda.cpp (Cuda::device_synchronize).
 * ---------------------------------------------------------------------- */
NBLAHIP_EXPORT int nblahip_device_count(int *count);
NBLAHIP_EXPORT int nblahip_set_device(int device);
NBLAHIP_EXPORT int nblahip_get_device(int *device);
NBLAHIP_EXPORT int nblahip_device_synchronize(void);
NBLAHIP_EXPORT int nblahip_stream_synchronize(void *stream);
/* name (up to name_len-1 chars), compute units, wavefront size, HBM bytes. */
NBLAHIP_EXPORT int nblahip_device_info(int device, char *name, size_t name_len,
                                       int *compute_units, int *wave_size,
                                       size_t *total_mem);
NBLAHIP_EXPORT int nblahip_malloc(void **ptr, size_t bytes);
NBLAHIP_EXPORT int nblahip_free(void *ptr);
/* Page-locked host memory (hipHostMalloc), the storage of the pinned host
 * array class (CudaCachedHostArray / CudaHostMemory,
 * include/nbla/cuda/array/cuda_array.hpp:92-108).  Copies to and from it are
 * direct DMA transfers. */
NBLAHIP_EXPORT int nblahip_host_malloc(void **ptr, size_t bytes);
NBLAHIP_EXPORT int nblahip_host_free(void *ptr);
NBLAHIP_EXPORT int nblahip_memcpy_h2d(void *dst, const void *src, size_t bytes,
                                      void *stream);
NBLAHIP_EXPORT int nblahip_memcpy_d2h(void *dst, const void *src, size_t bytes,
                                      void *stream);
NBLAHIP_EXPORT int nblahip_memcpy_d2d(void *dst, const void *src, size_t bytes,
                                      void *stream);
/* Asynchronous transfers (src/nbla/cuda/array/cuda_array.cpp:83-158: the
 * AsyncFlag::ASYNC synchronizers issue cudaMemcpyAsync on the backend's
 * stream_HtoD / stream_DtoH and order it against the null stream with events).
 * The *_async copies return without waiting and are meant for page-locked host
 * memory (nblahip_host_malloc); streams are created non-blocking with the
 * default priority, events without timing.  nblahip_event_query: *done = 1
 * when everything recorded before the event has finished. */
NBLAHIP_EXPORT int nblahip_memcpy_h2d_async(void *dst, const void *src,
                                            size_t bytes, void *stream);
NBLAHIP_EXPORT int nblahip_memcpy_d2h_async(void *dst, const void *src,
                                            size_t bytes, void *stream);
NBLAHIP_EXPORT int nblahip_stream_create(void **stream);
NBLAHIP_EXPORT int nblahip_stream_destroy(void *stream);
NBLAHIP_EXPORT int nblahip_event_create(void **event);
NBLAHIP_EXPORT int nblahip_event_destroy(void *event);
NBLAHIP_EXPORT int nblahip_event_record(void *event, void *stream);
NBLAHIP_EXPORT int nblahip_stream_wait_event(void *stream, void *event);
NBLAHIP_EXPORT int nblahip_event_synchronize(void *event);
NBLAHIP_EXPORT int nblahip_event_query(void *event, int *done);
NBLAHIP_EXPORT int nblahip_memset(void *dst, int byte, size_t bytes,
                                  void *stream);
/* dst[i] = (dst_dtype) src[i] for n elements (float32 <-> float16). */
NBLAHIP_EXPORT int nblahip_convert(void *dst, int dst_dtype, const void *src,
                                   int src_dtype, int64_t n, void *stream);
/* dst[i] = value for n elements of dtype. */
NBLAHIP_EXPORT int nblahip_fill(void *dst, int dtype, float value, int64_t n,
                                void *stream);
/* dst[i] = the low elem_bytes (1, 2, 4 or 8) bytes of pattern, for n elements:
 * the value fill of the array layer for the dtypes the functions here do not
 * compute in (CudaArray::fill covers every dtype through cuda_fill<T>,
 * include/nbla/cuda/array/cuda_array.cuh:44-55,99; the caller converts the
 * value to the element type). */
NBLAHIP_EXPORT int nblahip_fill_bytes(void *dst, int elem_bytes,
                                      unsigned long long pattern, int64_t n,
                                      void *stream);

/* Up to 16 small arrays converted between float16 and float32 in one launch:
 * dst[k][i] = (dst_dtype) src[k][i] for i < n[k] (arrays with n[k] == 0 are
 * skipped).  The normalization entry points take gamma, beta, statistics and
 * their gradients in float32; a "hip:half" graph that stores them in half
 * precision, as the reference's plain cuda:half type config does (Tc = half:
 * layer_normalization.cu:91-93, batch_normalization.cu:124-143), has its
 * Function classes stage them through this call - one launch before the
 * kernels for everything they read, one after for everything they wrote - so
 * the stored arrays keep their type. */
NBLAHIP_EXPORT int nblahip_stage_params(int count, const void *const *src,
                                        int src_dtype, void *const *dst,
                                        int dst_dtype, const int64_t *n,
                                        void *stream);

/* Axis permutation of a contiguous tensor (float32 or float16):
 *   dst[i_perm[0], ..., i_perm[ndim-1]] = src[i_0, ..., i_{ndim-1}]
 * i.e. axis k of dst is axis perm[k] of src, whose extents are shape[0..ndim-1]
 * (ndim <= 8); accum != 0 adds onto dst.  The Function classes use it for the
 * layouts the normalization kernels do not read in place; it replaces the
 * transposes of the core's ChannelFirstAdaptor the reference calls
 * (group_normalization.cu:40-55,93-109, instance_normalization.cu:40-51,81-94)
 * and its generic transpose kernel (kernel/transpose.cuh:19-53). */
NBLAHIP_EXPORT int nblahip_permute(const void *src, void *dst, int ndim,
                                   const int64_t *shape, const int *perm,
                                   int accum, int dtype, void *stream);

/* ------------------------------------------------------------------------
 * Per-kernel event timing, the counterpart of the reference's
 * CudaEventTimerCallback (python/src/nnabla_ext/cuda/utils/inspection/
 * profile.py:23-74), which brackets each function with CUDA events.  Here every
 * kernel launch carries its own start/stop event pair on the launch stream
 * (stamped at the begin and end of the kernel's execution).
 *   enable(n > 0): pre-create n event pairs and start recording (launches
 *                  beyond n are not recorded); enable(0): stop and release.
 *   reset        : forget the records, keep the pool.
 *   query        : wait for the recorded launches of `kernel_name` (the
 *                  __global__ function's name, e.g. "bn_bwd_apply_planes_kernel";
 *                  the row kernels are "row_fwd_kernel", "row_bwd_kernel_ln",
 *                  "row_bwd_kernel_in", "row_bwd_kernel_gn") and return their
 *                  summed duration and count.
 * Not for use while other threads are launching.
 * ---------------------------------------------------------------------- */
NBLAHIP_EXPORT int nblahip_profile_enable(int max_records);
NBLAHIP_EXPORT int nblahip_profile_reset(void);
NBLAHIP_EXPORT int nblahip_profile_query(const char *kernel_name,
                                         double *total_ms, int64_t *launches);
/* Names of the kernels recorded since the last reset, one per line, each once,
 * in order of first launch.  Writes at most `capacity` bytes (terminated);
 * *needed = bytes for the whole list. */
NBLAHIP_EXPORT int nblahip_profile_kernels(char *names, size_t capacity,
                                           size_t *needed);

/* ------------------------------------------------------------------------
 * Plan knobs.  Which kernel family serves a shape is decided per call from a
 * few integers (block counts per CU, size limits of the on-chip paths, on/off
 * switches of each specialised plan).  Every one has a default; the environment
 * variable NBLAHIP_<NAME> (read once, at the knob's first use) overrides the
 * default and nblahip_tune_set overrides both, from the next call on.  Results
 * never depend on a knob beyond the summation order of partial sums.  No
 * counterpart in the reference, whose launch shapes are compile-time macros
 * (include/nbla/cuda/common.hpp:337-343: NBLA_CUDA_NUM_THREADS,
 * NBLA_CUDA_GET_BLOCKS).
 *   set(name, value >= 0): override; set(name, -1): back to environment/default.
 *   get(name, fallback)  : the value a launch would use now.
 *   reset()              : drop every override made through set.
 * `name` is the knob without the NBLAHIP_ prefix, e.g. "BN_ONCHIP".
 * ---------------------------------------------------------------------- */
NBLAHIP_EXPORT int nblahip_tune_set(const char *name, int value);
NBLAHIP_EXPORT int nblahip_tune_get(const char *name, int fallback);
NBLAHIP_EXPORT int nblahip_tune_reset(void);

/* Testing aid, no counterpart in the reference.  The kernels whose blocks
 * exchange partial sums tag every exchanged word with a per-launch epoch, a
 * 32-bit counter per GPU; when it wraps (after 2^32 such launches) the library
 * waits for the device, clears its exchange array and starts over at 1.  This
 * sets the counter of the current device so that a test can walk it across
 * the wrap. */
NBLAHIP_EXPORT int nblahip_xchg_set_epoch(unsigned int epoch);

#ifdef __cplusplus
}
#endif
#endif /* NBLAHIP_H_ */
