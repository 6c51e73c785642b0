// The backend singleton of the "hip" context: device bookkeeping and the
// caching device allocator behind HipCachedArray.  Slim counterpart of the
// reference's `Cuda` singleton (include/nbla/cuda/cuda.hpp:49-187,
// src/nbla/cuda/cuda.cpp:30-338): no BLAS/RNG handles and one stream (the
// null stream every reference kernel launches on).
#pragma once

#include <map>
#include <mutex>
#include <nbla/backend_registry.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/singleton_manager.hpp>

namespace nbla {

class NBLA_HIP_API Hip : public BackendBase {
public:
  Hip();
  ~Hip();
  vector<string> array_classes() const override;
  void device_synchronize(const string &device) override;
  void default_stream_synchronize(const string &device) override;

  // Caching allocator: freed blocks are kept per (device, rounded size) and
  // handed out again without touching the driver; requests are rounded up to
  // 512 bytes (the reference's alignment, src/nbla/cuda/memory/cuda_memory.cpp:51-75).
  void *alloc(size_t bytes, int device);
  void free(void *ptr, size_t bytes, int device);
  // Returns cached blocks to the driver (all devices).
  void free_unused_device_caches();
  size_t cached_bytes() const;
  size_t live_bytes() const;

private:
  mutable std::mutex mu_;
  std::map<std::pair<int, size_t>, vector<void *>> cache_;
  size_t cached_bytes_ = 0, live_bytes_ = 0;
};

} // namespace nbla
