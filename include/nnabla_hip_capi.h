/*
 * nnabla_hip_capi.h - flat C surface over the "hip" backend's C++ layer
 * (libnnabla_hip.so): initialisation, Variables, and the four normalization
 * Functions created through the function registry by context, exactly the
 * calls a language binding makes.  It plays the part of the reference's
 * Cython layer (python/src/nnabla_ext/cuda/init.pyx:28-71 calls init_cuda()
 * and registers the context; the core's function bindings then create
 * functions by name and context).  Errors of the C++ layer (nbla::Exception)
 * are caught here: functions return 0 on success and non-zero otherwise, and
 * nnabla_hip_last_error() returns the message of the calling thread's last
 * failure.
 */
#ifndef NNABLA_HIP_CAPI_H_
#define NNABLA_HIP_CAPI_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNABLA_HIP_EXPORT __attribute__((visibility("default")))

typedef struct nnabla_hip_variable nnabla_hip_variable;
typedef struct nnabla_hip_function nnabla_hip_function;

/* nbla::init_hip() (idempotent). */
NNABLA_HIP_EXPORT int nnabla_hip_init(void);
NNABLA_HIP_EXPORT const char *nnabla_hip_last_error(void);
/* Array classes of the backend, comma separated ("HipCachedArray,HipArray"). */
NNABLA_HIP_EXPORT const char *nnabla_hip_array_classes(void);
NNABLA_HIP_EXPORT int nnabla_hip_device_synchronize(const char *device_id);
/* Bytes held by live device arrays / kept in the allocator cache. */
NNABLA_HIP_EXPORT int nnabla_hip_device_count(int *count);
/* Host array class variable_set/get stage through: "CpuArray" (default) or
 * "HipCachedHostArray" (page-locked memory, direct DMA transfers). */
NNABLA_HIP_EXPORT int nnabla_hip_set_host_array_class(const char *name);
NNABLA_HIP_EXPORT int nnabla_hip_memory_stats(uint64_t *live_bytes, uint64_t *cached_bytes);
NNABLA_HIP_EXPORT int nnabla_hip_clear_memory_cache(void);

/* Variables.  which: 0 = data, 1 = grad.  dtype: 0 = float32, 1 = float16
 * (the host buffer is always float32; float16 storage rounds to nearest). */
NNABLA_HIP_EXPORT nnabla_hip_variable *nnabla_hip_variable_new(int ndim, const int64_t *shape);
NNABLA_HIP_EXPORT void nnabla_hip_variable_delete(nnabla_hip_variable *v);
NNABLA_HIP_EXPORT int nnabla_hip_variable_ndim(nnabla_hip_variable *v);
NNABLA_HIP_EXPORT int nnabla_hip_variable_shape(nnabla_hip_variable *v, int64_t *shape_out);
NNABLA_HIP_EXPORT int nnabla_hip_variable_set(nnabla_hip_variable *v, int which, const float *host,
                                              int64_t n, int dtype);
NNABLA_HIP_EXPORT int nnabla_hip_variable_get(nnabla_hip_variable *v, int which, float *host,
                                              int64_t n);
/* NdArray::cast(dtype, Context({}, array_class, device_id), write_only,
 * async_flags): moves the variable's content into an array of that class.
 * async_flags as the core's AsyncFlag (1 = ASYNC, 2 = UNSAFE): with ASYNC and a
 * page-locked host array on the other side the transfer is enqueued on the
 * backend's transfer stream and the call returns at once
 * (src/nbla/cuda/array/cuda_array.cpp:83-158); the next use of the array waits
 * for it.  nnabla_hip_pending_transfers: host-to-device transfers whose source
 * array the backend still keeps alive. */
NNABLA_HIP_EXPORT int nnabla_hip_variable_cast(nnabla_hip_variable *v, int which,
                                               const char *array_class, const char *device_id,
                                               int dtype, int write_only, int async_flags);
/* dtype above: 0 float, 1 half, or 0x100 + the core's dtypes enumerator (BOOL 0,
 * BYTE 1, UBYTE 2, SHORT 3, USHORT 4, INT 5, UINT 6, LONG 7, ULONG 8, FLOAT 9,
 * DOUBLE 10, HALF 23): device arrays store and copy every dtype, as CudaArray
 * does (src/nbla/cuda/array/cuda_array.cpp:211-279); only float and half are
 * filled with values and converted.  set_raw / get_raw move n elements of that
 * dtype between host memory and the variable without conversion. */
NNABLA_HIP_EXPORT int nnabla_hip_variable_set_raw(nnabla_hip_variable *v, int which,
                                                  const void *host, int64_t n, int dtype);
NNABLA_HIP_EXPORT int nnabla_hip_variable_get_raw(nnabla_hip_variable *v, int which, void *host,
                                                  int64_t n, int dtype);
NNABLA_HIP_EXPORT int nnabla_hip_pending_transfers(uint64_t *count);
NNABLA_HIP_EXPORT int nnabla_hip_variable_zero(nnabla_hip_variable *v, int which);
NNABLA_HIP_EXPORT int nnabla_hip_variable_fill(nnabla_hip_variable *v, int which, float value);
/* dtype the variable's up-to-date array is stored in (codes as above: 0 float,
 * 1 half, 0x100 + n otherwise), -1 when it holds nothing yet (never written,
 * or zeroed / filled lazily). */
NNABLA_HIP_EXPORT int nnabla_hip_variable_stored_dtype(nnabla_hip_variable *v, int which,
                                                       int *dtype);

/* Function creation through the registry.  `backends` is the context's backend
 * preference list, comma separated (e.g. "hip:half,hip:float"). */
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_batch_normalization(
    const char *backends, const char *array_class, const char *device_id, const int *axes,
    int n_axes, float decay_rate, float eps, int batch_stat, int no_scale, int no_bias);
/* inputs [x, beta, gamma, mean, var] or [x, beta, gamma, mean, var, z];
 * nonlinearity must be "relu". */
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_fused_batch_normalization(
    const char *backends, const char *array_class, const char *device_id, const int *axes,
    int n_axes, float decay_rate, float eps, int batch_stat, const char *nonlinearity);
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_layer_normalization(
    const char *backends, const char *array_class, const char *device_id, const int *batch_axis,
    int n_batch_axis, float eps, int no_scale, int no_bias);
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_group_normalization(
    const char *backends, const char *array_class, const char *device_id, int num_groups,
    int channel_axis, const int *batch_axis, int n_batch_axis, float eps, int no_scale,
    int no_bias);
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_instance_normalization(
    const char *backends, const char *array_class, const char *device_id, int channel_axis,
    const int *batch_axis, int n_batch_axis, float eps, int no_scale, int no_bias);
/* TensorNormalizationCuda / WeightStandardizationCuda
 * (include/nbla/cuda/function/tensor_normalization.hpp:22-46,
 * weight_standardization.hpp:22-46).  axes: the axes the statistics keep,
 * read in place when adjacent, gathered by a device permutation otherwise (the
 * reference's composite transposes for such sets). */
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_tensor_normalization(
    const char *backends, const char *array_class, const char *device_id, const int *axes,
    int n_axes, float eps, int no_scale, int no_bias);
NNABLA_HIP_EXPORT nnabla_hip_function *nnabla_hip_create_weight_standardization(
    const char *backends, const char *array_class, const char *device_id, int channel_axis,
    float eps);
NNABLA_HIP_EXPORT void nnabla_hip_function_delete(nnabla_hip_function *f);
NNABLA_HIP_EXPORT const char *nnabla_hip_function_name(nnabla_hip_function *f);

/* Function::setup / forward / backward / recompute. */
NNABLA_HIP_EXPORT int nnabla_hip_function_setup(nnabla_hip_function *f,
                                                nnabla_hip_variable **inputs, int n_inputs,
                                                nnabla_hip_variable **outputs, int n_outputs);
NNABLA_HIP_EXPORT int nnabla_hip_function_forward(nnabla_hip_function *f,
                                                  nnabla_hip_variable **inputs, int n_inputs,
                                                  nnabla_hip_variable **outputs, int n_outputs);
NNABLA_HIP_EXPORT int nnabla_hip_function_recompute(nnabla_hip_function *f,
                                                    nnabla_hip_variable **inputs, int n_inputs,
                                                    nnabla_hip_variable **outputs, int n_outputs);
NNABLA_HIP_EXPORT int nnabla_hip_function_backward(nnabla_hip_function *f,
                                                   nnabla_hip_variable **inputs, int n_inputs,
                                                   nnabla_hip_variable **outputs, int n_outputs,
                                                   const int *propagate_down, const int *accum);

#ifdef __cplusplus
}
#endif
#endif /* NNABLA_HIP_CAPI_H_ */
