// The backend singleton of the "hip" context: device bookkeeping and the
// caching device allocator behind HipCachedArray.  Slim counterpart of the
// reference's `Cuda` singleton (include/nbla/cuda/cuda.hpp:49-187,
// src/nbla/cuda/cuda.cpp:30-338): no BLAS/RNG handles and one stream (the
// null stream every reference kernel launches on).
#pragma once

#include <map>
#include <memory>
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

  // Transfer streams of a device, one per direction (the reference's
  // stream_HtoD / stream_DtoH, include/nbla/cuda/cuda.hpp:118-119): created on
  // first use, non-blocking, default priority.
  void *transfer_stream(int device, bool to_device);
  // Keeps `event` (and with it the source array of its transfer) alive until
  // the transfer has finished; finished ones are dropped on later calls and by
  // device_synchronize.
  void keep_until_done(std::shared_ptr<class HipEvent> event);
  size_t pending_transfers();

private:
  void reap_locked();
  std::map<std::pair<int, bool>, void *> streams_;
  vector<std::shared_ptr<class HipEvent>> pending_;
  mutable std::mutex mu_;
  std::map<std::pair<int, size_t>, vector<void *>> cache_;
  size_t cached_bytes_ = 0, live_bytes_ = 0;
};

} // namespace nbla
