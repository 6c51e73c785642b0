// The exchange array of xchg.cuh and the per-launch epochs.
#include <atomic>
#include <mutex>

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
// Launch epochs and ring positions, per device, under one lock (a launch takes
// it for a few instructions; the clearing at an epoch wrap holds it throughout).
std::mutex g_mu;
uint32_t g_epoch[kMaxDevices];
uint64_t g_ring[kMaxDevices];

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
  std::lock_guard<std::mutex> lock(g_mu);
  // Epochs are never 0 (the array starts zeroed) and count up per launch.
  // When the 32-bit counter wraps - after 2^32 launches on this GPU - a word
  // that an old launch reserved and never overwrote could carry the epoch of a
  // new one, so the array is cleared once, with the device idle before and
  // after (the only host synchronisation in this library, every 4 billion
  // launches); launches of other threads wait on the lock meanwhile.
  if (++g_epoch[dev] == 0) {
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemset(base, 0, kXchgWords * sizeof(unsigned long long));
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
      *status = static_cast<int>(e);
      --g_epoch[dev]; // the next launch tries again
      return false;
    }
    g_ring[dev] = 0;
    g_epoch[dev] = 1;
  }
  *epoch = g_epoch[dev];
  // A region never wraps around the end of the ring: one that would starts at
  // word 0 and the ring position moves behind it, so regions of consecutive
  // launches stay disjoint until the ring has gone round once (then a word that
  // a launch still in flight loses to a newer one fails the epoch test and its
  // reader recomputes the value).
  uint64_t at = g_ring[dev] % kXchgWords;
  if (at + words > kXchgWords) at = 0;
  g_ring[dev] = at + words;
  *region = base + at;
  return true;
}

void xchg_debug_set_epoch(int dev, uint32_t epoch) {
  if (dev < 0 || dev >= kMaxDevices) return;
  std::lock_guard<std::mutex> lock(g_mu);
  g_epoch[dev] = epoch;
}

} // namespace nblahip
