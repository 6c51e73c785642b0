// HipArray / HipCachedArray and the host<->device synchronizers.
#include <nbla/hip/array/hip_array.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

HipArray::HipArray(Size_t size, dtypes dtype, const Context &ctx, bool cached)
    : Array(size, dtype, ctx), device_(std::stoi(ctx.device_id)), cached_(cached) {
  hip_dtype_code(dtype); // rejects unsupported dtypes up front
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

void HipArray::zero() {
  hip_set_device(device_);
  NBLA_HIP_CHECK(nblahip_fill(ptr_, hip_dtype_code(dtype_), 0.f, size_, nullptr));
}

void HipArray::fill(float value) {
  hip_set_device(device_);
  NBLA_HIP_CHECK(nblahip_fill(ptr_, hip_dtype_code(dtype_), value, size_, nullptr));
}

void HipArray::copy_from(const Array *src) {
  NBLA_CHECK(src->size() == size_, error_code::value, "size mismatch in HipArray::copy_from");
  hip_set_device(device_);
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

void synchronizer_hip_array_cpu_array(Array *src, Array *dst) {
  NBLA_CHECK(src->size() == dst->size() && src->dtype() == dst->dtype(), error_code::value,
             "device-to-host copy needs equal size and dtype");
  hip_set_device(static_cast<HipArray *>(src)->device());
  NBLA_HIP_CHECK(nblahip_memcpy_d2h(dst->pointer<void>(), src->const_pointer<void>(), src->nbytes(),
                                    nullptr));
}

void synchronizer_cpu_array_hip_array(Array *src, Array *dst) {
  NBLA_CHECK(src->size() == dst->size() && src->dtype() == dst->dtype(), error_code::value,
             "host-to-device copy needs equal size and dtype");
  hip_set_device(static_cast<HipArray *>(dst)->device());
  NBLA_HIP_CHECK(nblahip_memcpy_h2d(dst->pointer<void>(), src->const_pointer<void>(), src->nbytes(),
                                    nullptr));
}

} // namespace nbla
