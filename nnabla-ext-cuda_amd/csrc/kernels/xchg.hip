// The exchange array of xchg.cuh and the per-launch epochs.
#include <atomic>

#include "launch.hpp"
#include "xchg.cuh"

namespace nblahip {

namespace {

// A ring inside the library's own data segment: zero when the code object is
// loaded and from then on written only through xchg_publish, which is what
// makes an epoch match proof of publication.  One array per GPU.
constexpr size_t kXchgWords = size_t{1} << 19; // 4 MiB
constexpr int kMaxDevices = 64;
__device__ __align__(256) unsigned long long xchg_words[kXchgWords];
std::atomic<unsigned long long *> g_base[kMaxDevices];
std::atomic<uint32_t> g_epoch[kMaxDevices];
std::atomic<uint64_t> g_ring[kMaxDevices];

} // namespace

size_t xchg_capacity() { return kXchgWords; }

bool xchg_acquire(size_t words, hipStream_t stream, unsigned long long **region, uint32_t *epoch,
                  int *status) {
  *status = 0;
  if (words == 0 || words > kXchgWords) return false;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (cap != hipStreamCaptureStatusNone) return false;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
  unsigned long long *base = g_base[dev].load(std::memory_order_acquire);
  if (!base) {
    void *p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(xchg_words)); e != hipSuccess || !p) {
      *status = e != hipSuccess ? static_cast<int>(e) : static_cast<int>(hipErrorInvalidSymbol);
      return false;
    }
    base = static_cast<unsigned long long *>(p);
    g_base[dev].store(base, std::memory_order_release);
  }
  // Never 0 (the array starts zeroed).  Regions of launches in flight at the
  // same time may overlap once the ring wraps; an overwritten word fails the
  // epoch test and its reader recomputes the value.
  uint32_t ep = g_epoch[dev].fetch_add(1, std::memory_order_relaxed) + 1;
  if (ep == 0) ep = g_epoch[dev].fetch_add(1, std::memory_order_relaxed) + 1;
  *epoch = ep;
  const uint64_t at = g_ring[dev].fetch_add(words, std::memory_order_relaxed) % kXchgWords;
  *region = base + (at + words <= kXchgWords ? at : 0);
  return true;
}

} // namespace nblahip
