// Exchange of single floats between the workgroups of one launch without a
// barrier, a fence or zeroed memory.
//
// A value travels as one 64-bit word {value, epoch}, written and read with
// relaxed device-scope atomics.  `epoch` is unique per launch and the words
// live in an array inside the library that starts zeroed and only ever holds
// such words, so a word that carries this launch's epoch holds the value its
// producer wrote for it, and any other word does not count.  A consumer polls
// a word a bounded number of times; what it does when the word does not turn
// up (the producer is not scheduled yet, or another launch overwrote the slot)
// is its own business - the kernels here recompute the value themselves, so
// every wave reaches the end of its kernel whatever the other blocks do.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nblahip {

__device__ __forceinline__ void xchg_publish(unsigned long long *slot, float v, uint32_t epoch) {
  const unsigned long long w = (static_cast<unsigned long long>(epoch) << 32) | __float_as_uint(v);
  __hip_atomic_store(slot, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// true and *v set once the word carries `epoch`; false after `spin` polls.
__device__ __forceinline__ bool xchg_poll(const unsigned long long *slot, uint32_t epoch, int spin,
                                          float *v) {
  for (int it = 0; it < spin; ++it) {
    const unsigned long long w =
        __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (static_cast<uint32_t>(w >> 32) == epoch) {
      *v = __uint_as_float(static_cast<uint32_t>(w));
      return true;
    }
    __builtin_amdgcn_s_sleep(8);
  }
  return false;
}

// Two adjacent words at once (both loads in flight together: one round trip).
__device__ __forceinline__ bool xchg_poll2(const unsigned long long *slot, uint32_t epoch, int spin,
                                           float *v0, float *v1) {
  for (int it = 0; it < spin; ++it) {
    const unsigned long long w0 =
        __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long w1 =
        __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (static_cast<uint32_t>(w0 >> 32) == epoch && static_cast<uint32_t>(w1 >> 32) == epoch) {
      *v0 = __uint_as_float(static_cast<uint32_t>(w0));
      *v1 = __uint_as_float(static_cast<uint32_t>(w1));
      return true;
    }
    __builtin_amdgcn_s_sleep(8);
  }
  return false;
}

// Host side (xchg.hip): a region of `words` exchange words on the current
// device and a fresh epoch for one launch on `stream`.  Returns false when the
// launch must not use the exchange: the stream is being captured (a replayed
// launch would reuse its epoch), or the region exceeds the array.
bool xchg_acquire(size_t words, hipStream_t stream, unsigned long long **region, uint32_t *epoch,
                  int *status);
// Most words one launch may ask for.
size_t xchg_capacity();
// Testing aid: the epoch the next launch on device `dev` continues from.
void xchg_debug_set_epoch(int dev, uint32_t epoch);

} // namespace nblahip
