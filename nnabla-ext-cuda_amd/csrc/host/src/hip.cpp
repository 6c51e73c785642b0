// Hip backend singleton and device helpers.
#include <nbla/hip/array/hip_array.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

void hip_set_device(int device) { NBLA_HIP_CHECK(nblahip_set_device(device)); }

int hip_get_device() {
  int d = 0;
  NBLA_HIP_CHECK(nblahip_get_device(&d));
  return d;
}

Hip::Hip() {}

Hip::~Hip() {
  pending_.clear();
  for (auto &kv : streams_) NBLA_HIP_FORCE_ASSERT(nblahip_stream_destroy(kv.second));
  for (auto &kv : cache_)
    for (void *p : kv.second) NBLA_HIP_FORCE_ASSERT(nblahip_free(p));
}

vector<string> Hip::array_classes() const { return {"HipCachedArray", "HipArray"}; }

void Hip::device_synchronize(const string &device) {
  hip_set_device(std::stoi(device));
  NBLA_HIP_CHECK(nblahip_device_synchronize());
  std::lock_guard<std::mutex> lock(mu_);
  reap_locked();
}

void *Hip::transfer_stream(int device, bool to_device) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = streams_.find(std::make_pair(device, to_device));
  if (it != streams_.end()) return it->second;
  hip_set_device(device);
  void *st = nullptr;
  NBLA_HIP_CHECK(nblahip_stream_create(&st));
  streams_[std::make_pair(device, to_device)] = st;
  return st;
}

void Hip::reap_locked() {
  size_t kept = 0;
  for (auto &e : pending_) {
    int done = 0;
    if (nblahip_event_query(e->raw_event(), &done) == 0 && done) continue;
    pending_[kept++] = e;
  }
  pending_.resize(kept);
}

void Hip::keep_until_done(std::shared_ptr<HipEvent> event) {
  std::lock_guard<std::mutex> lock(mu_);
  reap_locked();
  pending_.push_back(event);
}

size_t Hip::pending_transfers() {
  std::lock_guard<std::mutex> lock(mu_);
  reap_locked();
  return pending_.size();
}

void Hip::default_stream_synchronize(const string &device) {
  hip_set_device(std::stoi(device));
  NBLA_HIP_CHECK(nblahip_stream_synchronize(nullptr));
}

static size_t round_up_512(size_t bytes) { return (std::max<size_t>(bytes, 1) + 511) / 512 * 512; }

void *Hip::alloc(size_t bytes, int device) {
  const size_t rounded = round_up_512(bytes);
  {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = cache_.find(std::make_pair(device, rounded));
    if (it != cache_.end() && !it->second.empty()) {
      void *p = it->second.back();
      it->second.pop_back();
      cached_bytes_ -= rounded;
      live_bytes_ += rounded;
      return p;
    }
  }
  hip_set_device(device);
  void *p = nullptr;
  int status = nblahip_malloc(&p, rounded);
  if (status != 0) {
    // Out of memory: give the cache back to the driver and retry once, as the
    // reference's caching allocator does.
    free_unused_device_caches();
    status = nblahip_malloc(&p, rounded);
  }
  NBLA_CHECK(status == 0, error_code::memory, "device allocation of %zu bytes failed: %s", rounded,
             nblahip_error_string(status));
  std::lock_guard<std::mutex> lock(mu_);
  live_bytes_ += rounded;
  return p;
}

void Hip::free(void *ptr, size_t bytes, int device) {
  if (!ptr) return;
  const size_t rounded = round_up_512(bytes);
  std::lock_guard<std::mutex> lock(mu_);
  cache_[std::make_pair(device, rounded)].push_back(ptr);
  cached_bytes_ += rounded;
  live_bytes_ -= rounded;
}

void Hip::free_unused_device_caches() {
  std::map<std::pair<int, size_t>, vector<void *>> taken;
  {
    std::lock_guard<std::mutex> lock(mu_);
    taken.swap(cache_);
    cached_bytes_ = 0;
  }
  for (auto &kv : taken) {
    if (kv.second.empty()) continue;
    NBLA_HIP_FORCE_ASSERT(nblahip_set_device(kv.first.first));
    for (void *p : kv.second) NBLA_HIP_FORCE_ASSERT(nblahip_free(p));
  }
}

size_t Hip::cached_bytes() const {
  std::lock_guard<std::mutex> lock(mu_);
  return cached_bytes_;
}
size_t Hip::live_bytes() const {
  std::lock_guard<std::mutex> lock(mu_);
  return live_bytes_;
}

} // namespace nbla
