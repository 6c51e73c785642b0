// Device array classes of the "hip" backend: HipArray (driver allocation per
// array) and HipCachedArray (through the Hip singleton's caching allocator),
// plus the host<->device synchronizers.  Counterpart of the reference's
// CudaArray / CudaCachedArray (include/nbla/cuda/array/cuda_array.hpp:36-49,
// src/nbla/cuda/array/cuda_array.cpp:42-347).
#pragma once

#include <nbla/array.hpp>
#include <nbla/hip/common.hpp>

namespace nbla {

class NBLA_HIP_API HipArray : public Array {
protected:
  int device_;
  bool cached_;

public:
  HipArray(Size_t size, dtypes dtype, const Context &ctx, bool cached = false);
  ~HipArray() override;
  void zero() override;
  void fill(float value) override;
  void copy_from(const Array *src) override; // device-side, converts float32 <-> float16
  int device() const { return device_; }
};

class NBLA_HIP_API HipCachedArray : public HipArray {
public:
  HipCachedArray(Size_t size, dtypes dtype, const Context &ctx) : HipArray(size, dtype, ctx, true) {}
};

// Host array in page-locked memory (counterpart of CudaCachedHostArray,
// include/nbla/cuda/array/cuda_array.hpp:92-108): behaves as a CpuArray, and
// transfers between it and the device arrays are direct DMA copies.
class NBLA_HIP_API HipCachedHostArray : public CpuArray {
public:
  HipCachedHostArray(Size_t size, dtypes dtype, const Context &ctx);
  ~HipCachedHostArray() override;
  static Context filter_context(const Context &ctx) {
    return Context({}, "HipCachedHostArray", "");
  }
};

// Blocking copies between a host array and a device array of the same dtype.
NBLA_HIP_API void synchronizer_hip_array_cpu_array(Array *src, Array *dst);
NBLA_HIP_API void synchronizer_cpu_array_hip_array(Array *src, Array *dst);

} // namespace nbla
