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

// Copies between a host array and a device array of the same dtype
// (src/nbla/cuda/array/cuda_array.cpp:83-235).  Blocking by default.  With
// AsyncFlag::ASYNC and a page-locked host array (HipCachedHostArray) the copy is
// enqueued on the backend's transfer stream of its direction, after whatever
// the function stream (the null stream) holds at that moment, and recorded as
// an event in the destination array: the next cast / get of that array makes
// the function stream wait for it (and the host too, when the consumer is a
// host context and passes neither ASYNC nor UNSAFE).  A host-to-device copy
// keeps its source array alive until it has run unless AsyncFlag::UNSAFE is
// given.  Pageable host memory (CpuArray) is always copied with blocking
// semantics, whatever the flags say.
NBLA_HIP_API void synchronizer_hip_array_cpu_array(Array *src, Array *dst, const int async_flags);
NBLA_HIP_API void synchronizer_cpu_array_hip_array(Array *src, Array *dst, const int async_flags);

// A transfer enqueued on one of the backend's transfer streams (counterpart of
// CudaEvent, src/nbla/cuda/event.cpp:20-60).  Holds the source array so that it
// outlives the transfer for as long as the destination remembers the event.
class NBLA_HIP_API HipEvent : public Event {
  void *raw_event_;
  ArrayPtr src_;
  int device_;

public:
  HipEvent(void *raw_event, ArrayPtr src, int device)
      : raw_event_(raw_event), src_(src), device_(device) {}
  ~HipEvent() override;
  void *raw_event() { return raw_event_; }
  void wait_event(const Context ctx, const int async_flags = AsyncFlag::NONE) override;
};

} // namespace nbla
