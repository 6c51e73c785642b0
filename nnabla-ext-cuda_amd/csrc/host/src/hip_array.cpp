// HipArray / HipCachedArray and the host<->device synchronizers.
#include <nbla/hip/array/hip_array.hpp>
#include <nbla/hip/hip.hpp>

#include <cstring>

namespace nbla {

HipArray::HipArray(Size_t size, dtypes dtype, const Context &ctx, bool cached)
    : Array(size, dtype, ctx), device_(std::stoi(ctx.device_id)), cached_(cached) {
  if (cached_) {
    ptr_ = SingletonManager::get<Hip>()->alloc(nbytes(), device_);
  } else {
    hip_set_device(device_);
    NBLA_HIP_CHECK(nblahip_malloc(&ptr_, std::max<size_t>(nbytes(), 1)));
  }
}

HipArray::~HipArray() {
  if (!ptr_) return;
  if (cached_) {
    SingletonManager::get<Hip>()->free(ptr_, nbytes(), device_);
  } else {
    NBLA_HIP_FORCE_ASSERT(nblahip_free(ptr_));
  }
}

namespace {
bool is_float_dtype(dtypes d) { return d == dtypes::FLOAT || d == dtypes::HALF; }
} // namespace

// Any dtype is stored, moved and filled (the reference's CudaArray holds every
// dtype, src/nbla/cuda/array/cuda_array.cpp:211-279); conversions exist for
// the two float types the normalization functions compute in.
void HipArray::zero() {
  hip_set_device(device_);
  if (is_float_dtype(dtype_)) {
    NBLA_HIP_CHECK(nblahip_fill(ptr_, hip_dtype_code(dtype_), 0.f, size_, nullptr));
  } else {
    NBLA_HIP_CHECK(nblahip_memset(ptr_, 0, nbytes(), nullptr));
  }
}

namespace {
// `value` converted to the element type as a C++ cast does, as raw bytes.
template <typename D> unsigned long long element_bits(float value) {
  const D d = static_cast<D>(value);
  unsigned long long bits = 0;
  std::memcpy(&bits, &d, sizeof(D));
  return bits;
}
unsigned long long fill_pattern(dtypes dtype, float value) {
  switch (dtype) {
  case dtypes::BOOL: return value != 0.f ? 1u : 0u;
  case dtypes::BYTE: return element_bits<int8_t>(value);
  case dtypes::UBYTE: return element_bits<uint8_t>(value);
  case dtypes::SHORT: return element_bits<int16_t>(value);
  case dtypes::USHORT: return element_bits<uint16_t>(value);
  case dtypes::INT: return element_bits<int32_t>(value);
  case dtypes::UINT: return element_bits<uint32_t>(value);
  case dtypes::LONG: return element_bits<int64_t>(value);
  case dtypes::ULONG: return element_bits<uint64_t>(value);
  case dtypes::DOUBLE: return element_bits<double>(value);
  default: NBLA_ERROR(error_code::type, "HipArray::fill: unknown dtype");
  }
}
} // namespace

void HipArray::fill(float value) {
  if (value == 0.f) return zero();
  hip_set_device(device_);
  if (is_float_dtype(dtype_)) {
    NBLA_HIP_CHECK(nblahip_fill(ptr_, hip_dtype_code(dtype_), value, size_, nullptr));
  } else {
    NBLA_HIP_CHECK(nblahip_fill_bytes(ptr_, static_cast<int>(sizeof_dtype(dtype_)),
                                      fill_pattern(dtype_, value), size_, nullptr));
  }
}

void HipArray::copy_from(const Array *src) {
  NBLA_CHECK(src->size() == size_, error_code::value, "size mismatch in HipArray::copy_from");
  hip_set_device(device_);
  if (src->dtype() == dtype_) {
    NBLA_HIP_CHECK(nblahip_memcpy_d2d(ptr_, src->const_pointer<void>(), nbytes(), nullptr));
    return;
  }
  NBLA_HIP_CHECK(nblahip_convert(ptr_, hip_dtype_code(dtype_), src->const_pointer<void>(),
                                 hip_dtype_code(src->dtype()), size_, nullptr));
}

namespace {
void *pinned_alloc(size_t bytes) {
  void *p = nullptr;
  NBLA_HIP_CHECK(nblahip_host_malloc(&p, std::max<size_t>(bytes, 1)));
  return p;
}
} // namespace

HipCachedHostArray::HipCachedHostArray(Size_t size, dtypes dtype, const Context &ctx)
    : CpuArray(size, dtype, ctx,
               pinned_alloc(static_cast<size_t>(size) * sizeof_dtype(dtype))) {}

HipCachedHostArray::~HipCachedHostArray() { NBLA_HIP_FORCE_ASSERT(nblahip_host_free(ptr_)); }

HipEvent::~HipEvent() { NBLA_HIP_FORCE_ASSERT(nblahip_event_destroy(raw_event_)); }

void HipEvent::wait_event(const Context ctx, const int async_flags) {
  hip_set_device(device_);
  // the function stream (the null stream) waits for the transfer
  NBLA_HIP_CHECK(nblahip_stream_wait_event(nullptr, raw_event_));
  // a host consumer that asked for neither ASYNC nor UNSAFE waits as well
  if (!(async_flags & AsyncFlag::ASYNC) && !(async_flags & AsyncFlag::UNSAFE) &&
      is_cpu_context(ctx)) {
    NBLA_HIP_CHECK(nblahip_stream_synchronize(nullptr));
  }
}

namespace {
bool is_pinned(const Array *a) { return dynamic_cast<const HipCachedHostArray *>(a) != nullptr; }

void check_pair(Array *src, Array *dst, const char *what) {
  NBLA_CHECK(src->size() == dst->size() && src->dtype() == dst->dtype(), error_code::value,
             "%s copy needs equal size and dtype", what);
}

// cuda_array.cpp:83-115 / :118-158: the transfer stream first waits for what
// the function stream holds now (the kernels that produce the source or still
// read the destination), then copies, then records the event the destination
// array keeps.
void enqueue_async(Array *src, Array *dst, bool to_device, int device, const int async_flags) {
  src->wait_event(dst->context(), async_flags);
  NBLA_CHECK(!dst->have_event(), error_code::target_specific_async,
             "Duplicated asynchronous memcpy to the same destination array");
  Hip *hip = SingletonManager::get<Hip>();
  void *stream = hip->transfer_stream(device, to_device);
  void *fence = nullptr;
  NBLA_HIP_CHECK(nblahip_event_create(&fence));
  int status = nblahip_event_record(fence, nullptr);
  if (status == 0) status = nblahip_stream_wait_event(stream, fence);
  NBLA_HIP_FORCE_ASSERT(nblahip_event_destroy(fence));
  NBLA_HIP_CHECK(status);
  void *event = nullptr;
  NBLA_HIP_CHECK(nblahip_event_create(&event));
  auto recorded = std::make_shared<HipEvent>(event, src->getptr(), device);
  if (to_device) {
    NBLA_HIP_CHECK(nblahip_memcpy_h2d_async(dst->pointer<void>(), src->const_pointer<void>(),
                                            src->nbytes(), stream));
  } else {
    NBLA_HIP_CHECK(nblahip_memcpy_d2h_async(dst->pointer<void>(), src->const_pointer<void>(),
                                            src->nbytes(), stream));
  }
  NBLA_HIP_CHECK(nblahip_event_record(event, stream));
  if (to_device && !(async_flags & AsyncFlag::UNSAFE)) {
    // Keeps the host source alive until the copy has run, also after the
    // destination has dropped the event (the reference hangs a delete guard on
    // a stream callback, cuda_array.cpp:146-151; here the backend keeps the
    // guard and drops it once the event reports completion).
    hip->keep_until_done(recorded);
  }
  dst->set_event(recorded);
}

void copy_blocking(Array *src, Array *dst, bool to_device, const int async_flags) {
  src->wait_event(dst->context(), async_flags);
  NBLA_CHECK(!dst->have_event(), error_code::target_specific_async,
             "Duplicated asynchronous memcpy to the same destination array");
  if (to_device) {
    NBLA_HIP_CHECK(nblahip_memcpy_h2d(dst->pointer<void>(), src->const_pointer<void>(),
                                      src->nbytes(), nullptr));
  } else {
    NBLA_HIP_CHECK(nblahip_memcpy_d2h(dst->pointer<void>(), src->const_pointer<void>(),
                                      src->nbytes(), nullptr));
  }
  dst->set_event(nullptr);
}
} // namespace

void synchronizer_hip_array_cpu_array(Array *src, Array *dst, const int async_flags) {
  check_pair(src, dst, "device-to-host");
  const int device = static_cast<HipArray *>(src)->device();
  hip_set_device(device);
  if ((async_flags & AsyncFlag::ASYNC) && is_pinned(dst)) {
    enqueue_async(src, dst, false, device, async_flags);
  } else {
    copy_blocking(src, dst, false, async_flags);
  }
}

void synchronizer_cpu_array_hip_array(Array *src, Array *dst, const int async_flags) {
  check_pair(src, dst, "host-to-device");
  const int device = static_cast<HipArray *>(dst)->device();
  hip_set_device(device);
  if ((async_flags & AsyncFlag::ASYNC) && is_pinned(src)) {
    enqueue_async(src, dst, true, device, async_flags);
  } else {
    copy_blocking(src, dst, true, async_flags);
  }
}

} // namespace nbla
