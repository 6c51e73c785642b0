// init_hip(): registration of the "hip" backend (src/nbla/cuda/init.cpp.tmpl:65-270
// is the reference's equivalent; here the table is five functions by two type
// configs, written out by hand instead of generated from yaml).
#include <mutex>

#include <nbla/cpu.hpp>
#include <nbla/function_registry.hpp>
#include <nbla/hip/array/hip_array.hpp>
#include <nbla/hip/function/batch_normalization.hpp>
#include <nbla/hip/function/fused_batch_normalization.hpp>
#include <nbla/hip/function/group_normalization.hpp>
#include <nbla/hip/function/instance_normalization.hpp>
#include <nbla/hip/function/layer_normalization.hpp>
#include <nbla/hip/function/tensor_normalization.hpp>
#include <nbla/hip/function/weight_standardization.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/init.hpp>

namespace nbla {

#ifdef NBLA_HIP_USE_CORE_STANDIN
// With the real core these registries live in libnnabla.
NBLA_REGISTER_FUNCTION_SOURCE(BatchNormalization, const vector<int> &, float, float, bool, bool, bool);
NBLA_REGISTER_FUNCTION_SOURCE(FusedBatchNormalization, const vector<int> &, float, float, bool,
                              const string &);
NBLA_REGISTER_FUNCTION_SOURCE(LayerNormalization, const vector<int> &, float, bool, bool);
NBLA_REGISTER_FUNCTION_SOURCE(GroupNormalization, int, int, const vector<int> &, float, bool, bool);
NBLA_REGISTER_FUNCTION_SOURCE(InstanceNormalization, int, const vector<int> &, float, bool, bool);
NBLA_REGISTER_FUNCTION_SOURCE(TensorNormalization, const vector<int> &, float, bool, bool);
NBLA_REGISTER_FUNCTION_SOURCE(WeightStandardization, int, float);
#endif

void init_hip() {
  static std::mutex mtx;
  static bool is_initialized = false;
  std::lock_guard<std::mutex> lock(mtx);
  if (is_initialized) return;

  init_cpu();

  // Backend
  NBLA_REGISTER_BACKEND("hip", [] { return static_cast<BackendBase *>(SingletonManager::get<Hip>()); });

  // Array classes and synchronizers
  ArrayCreator::add_creator("HipArray", [](Size_t s, dtypes d, const Context &c) -> Array * {
    return new HipArray(s, d, c);
  });
  ArrayCreator::add_creator("HipCachedArray", [](Size_t s, dtypes d, const Context &c) -> Array * {
    return new HipCachedArray(s, d, c);
  });
  ArrayCreator::add_creator("HipCachedHostArray", [](Size_t s, dtypes d, const Context &c) -> Array * {
    return new HipCachedHostArray(s, d, c);
  });
  // The pinned host array is a host array: plain copies to and from CpuArray -
  // once the source's pending transfer (an ASYNC device-to-host copy leaves a
  // HipEvent on the pinned array) has landed, as the reference's synchronizers
  // wait first (src/nbla/cuda/array/cuda_array.cpp:88,125,164).
  auto host_copy = [](Array *src, Array *dst, const int async_flags) {
    src->wait_event(dst->context(), async_flags & ~(AsyncFlag::ASYNC | AsyncFlag::UNSAFE));
    dst->copy_from(src);
  };
  ArraySynchronizer::add_synchronizer("HipCachedHostArray", "CpuArray", host_copy);
  ArraySynchronizer::add_synchronizer("CpuArray", "HipCachedHostArray", host_copy);
  ArraySynchronizer::add_synchronizer("HipCachedHostArray", "HipCachedHostArray", host_copy);
  const char *device_classes[] = {"HipArray", "HipCachedArray"};
  for (const char *dc : device_classes) {
    ArraySynchronizer::add_synchronizer(dc, "CpuArray", synchronizer_hip_array_cpu_array);
    ArraySynchronizer::add_synchronizer("CpuArray", dc, synchronizer_cpu_array_hip_array);
    ArraySynchronizer::add_synchronizer(dc, "HipCachedHostArray", synchronizer_hip_array_cpu_array);
    ArraySynchronizer::add_synchronizer("HipCachedHostArray", dc, synchronizer_cpu_array_hip_array);
    // device to device on the function stream, behind the source's pending upload
    for (const char *dc2 : device_classes)
      ArraySynchronizer::add_synchronizer(dc, dc2, [](Array *src, Array *dst, const int async_flags) {
        src->wait_event(dst->context(), async_flags);
        dst->copy_from(src);
      });
  }

  // Functions: same names as the reference registers, new backend key.
  typedef BatchNormalizationHip<float> BatchNormalizationHip_float;
  typedef BatchNormalizationHip<Half> BatchNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(BatchNormalization, BatchNormalizationHip_float, "hip:float",
                              const vector<int> &, float, float, bool, bool, bool);
  NBLA_REGISTER_FUNCTION_IMPL(BatchNormalization, BatchNormalizationHip_half, "hip:half",
                              const vector<int> &, float, float, bool, bool, bool);
  typedef FusedBatchNormalizationHip<float> FusedBatchNormalizationHip_float;
  typedef FusedBatchNormalizationHip<Half> FusedBatchNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(FusedBatchNormalization, FusedBatchNormalizationHip_float,
                              "hip:float", const vector<int> &, float, float, bool,
                              const string &);
  NBLA_REGISTER_FUNCTION_IMPL(FusedBatchNormalization, FusedBatchNormalizationHip_half, "hip:half",
                              const vector<int> &, float, float, bool, const string &);
  typedef LayerNormalizationHip<float> LayerNormalizationHip_float;
  typedef LayerNormalizationHip<Half> LayerNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(LayerNormalization, LayerNormalizationHip_float, "hip:float",
                              const vector<int> &, float, bool, bool);
  NBLA_REGISTER_FUNCTION_IMPL(LayerNormalization, LayerNormalizationHip_half, "hip:half",
                              const vector<int> &, float, bool, bool);
  typedef GroupNormalizationHip<float> GroupNormalizationHip_float;
  typedef GroupNormalizationHip<Half> GroupNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(GroupNormalization, GroupNormalizationHip_float, "hip:float", int, int,
                              const vector<int> &, float, bool, bool);
  NBLA_REGISTER_FUNCTION_IMPL(GroupNormalization, GroupNormalizationHip_half, "hip:half", int, int,
                              const vector<int> &, float, bool, bool);
  typedef InstanceNormalizationHip<float> InstanceNormalizationHip_float;
  typedef InstanceNormalizationHip<Half> InstanceNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(InstanceNormalization, InstanceNormalizationHip_float, "hip:float", int,
                              const vector<int> &, float, bool, bool);
  NBLA_REGISTER_FUNCTION_IMPL(InstanceNormalization, InstanceNormalizationHip_half, "hip:half", int,
                              const vector<int> &, float, bool, bool);
  typedef TensorNormalizationHip<float> TensorNormalizationHip_float;
  typedef TensorNormalizationHip<Half> TensorNormalizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(TensorNormalization, TensorNormalizationHip_float, "hip:float",
                              const vector<int> &, float, bool, bool);
  NBLA_REGISTER_FUNCTION_IMPL(TensorNormalization, TensorNormalizationHip_half, "hip:half",
                              const vector<int> &, float, bool, bool);
  typedef WeightStandardizationHip<float> WeightStandardizationHip_float;
  typedef WeightStandardizationHip<Half> WeightStandardizationHip_half;
  NBLA_REGISTER_FUNCTION_IMPL(WeightStandardization, WeightStandardizationHip_float, "hip:float",
                              int, float);
  NBLA_REGISTER_FUNCTION_IMPL(WeightStandardization, WeightStandardizationHip_half, "hip:half", int,
                              float);

  is_initialized = true;
}

} // namespace nbla
