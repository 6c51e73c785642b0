// Runtime shims of the C-ABI (device management, memory, dtype conversion)
// and the small host utilities shared by the launch code.
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.cuh"
#include "launch.hpp"
#include "xchg.cuh"

namespace nblahip {

int device_cus() {
  static std::mutex mu;
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lock(mu);
  if (cus[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    cus[dev] = v;
  }
  return cus[dev];
}

namespace {
// name -> value from the environment (-1: not set) and the value set through
// nblahip_tune_set (-1: none); the latter wins.
struct TuneEntry {
  int env = -1, set = -1;
};
std::mutex g_tune_mu;
std::unordered_map<std::string, TuneEntry> g_tune;

TuneEntry &tune_entry_locked(const char *name) {
  auto it = g_tune.find(name);
  if (it == g_tune.end()) {
    TuneEntry e;
    const std::string key = std::string("NBLAHIP_") + name;
    if (const char *s = std::getenv(key.c_str())) {
      char *end = nullptr;
      const long parsed = std::strtol(s, &end, 10);
      if (end != s && parsed >= 0 && parsed < (1 << 20)) e.env = static_cast<int>(parsed);
    }
    it = g_tune.emplace(name, e).first;
  }
  return it->second;
}
} // namespace

int tune_int(const char *name, int fallback) {
  // Only the environment's answer is cached: callers may pass different
  // fallbacks for the same knob.
  std::lock_guard<std::mutex> lock(g_tune_mu);
  const TuneEntry &e = tune_entry_locked(name);
  return e.set >= 0 ? e.set : e.env >= 0 ? e.env : fallback;
}

// ---------------------------------------------------------------------------
// Per-kernel event timing.
// ---------------------------------------------------------------------------
namespace {
struct ProfRecord {
  const char *tag;
  hipEvent_t start, stop;
};
struct ProfState {
  std::mutex mu;
  std::atomic<bool> enabled{false}; // read by launching threads without the lock
  std::vector<ProfRecord> records; // pool, events pre-created
  size_t used = 0;
  size_t dropped = 0;
} g_prof;
} // namespace

bool prof_acquire(const char *tag, hipEvent_t *start, hipEvent_t *stop) {
  if (!g_prof.enabled.load(std::memory_order_acquire)) return false;
  std::lock_guard<std::mutex> lock(g_prof.mu);
  if (g_prof.used >= g_prof.records.size()) {
    ++g_prof.dropped;
    return false;
  }
  ProfRecord &r = g_prof.records[g_prof.used++];
  r.tag = tag;
  *start = r.start;
  *stop = r.stop;
  return true;
}

static void prof_release_locked() {
  for (auto &r : g_prof.records) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_prof.records.clear();
  g_prof.used = 0;
  g_prof.dropped = 0;
}

template <typename D, typename S>
__global__ void __launch_bounds__(256)
convert_kernel(D *__restrict__ dst, const S *__restrict__ src, int64_t n) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll)
    dst[i] = from_f32<D>(to_f32<S>(src[i]));
}

template <typename D>
__global__ void __launch_bounds__(256) fill_kernel(D *__restrict__ dst, float v, int64_t n) {
  const D d = from_f32<D>(v);
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll) dst[i] = d;
}

template <typename W>
__global__ void __launch_bounds__(256) fill_words_kernel(W *__restrict__ dst, W v, int64_t n) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll) dst[i] = v;
}

// Several small arrays converted in one launch (blockIdx.y: the array).
constexpr int kStageMax = 16;
struct StageArgs {
  const void *src[kStageMax];
  void *dst[kStageMax];
  int64_t n[kStageMax];
};
template <typename D, typename S>
__global__ void __launch_bounds__(256) stage_params_kernel(const StageArgs a) {
  const int k = blockIdx.y;
  const S *__restrict__ src = static_cast<const S *>(a.src[k]);
  D *__restrict__ dst = static_cast<D *>(a.dst[k]);
  const int64_t n = a.n[k];
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll)
    dst[i] = from_f32<D>(to_f32<S>(src[i]));
}

static unsigned flat_grid(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return static_cast<unsigned>(b < 1 ? 1 : (b > 65536 ? 65536 : b));
}

} // namespace nblahip

using namespace nblahip;

static int hip_status(hipError_t e) { return e == hipSuccess ? 0 : static_cast<int>(e); }

extern "C" {

int nblahip_abi_version(void) { return 1; }

const char *nblahip_error_string(int code) {
  switch (code) {
  case NBLAHIP_OK: return "success";
  case NBLAHIP_EINVAL: return "nblahip: invalid argument (null pointer, negative size or unknown dtype)";
  case NBLAHIP_EWORKSPACE: return "nblahip: workspace is null, misaligned or too small";
  case NBLAHIP_ERANGE: return "nblahip: tensor has 2^31 or more elements";
  case NBLAHIP_EALIAS: return "nblahip: output overlaps an input";
  default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "nblahip: unknown status";
}

int nblahip_profile_enable(int max_records) {
  std::lock_guard<std::mutex> lock(g_prof.mu);
  g_prof.enabled = false;
  prof_release_locked();
  if (max_records <= 0) return 0;
  g_prof.records.reserve(static_cast<size_t>(max_records));
  for (int i = 0; i < max_records; ++i) {
    ProfRecord r{nullptr, nullptr, nullptr};
    hipError_t e = hipEventCreate(&r.start);
    if (e == hipSuccess) e = hipEventCreate(&r.stop);
    if (e != hipSuccess) {
      if (r.start) (void)hipEventDestroy(r.start);
      prof_release_locked();
      return static_cast<int>(e);
    }
    g_prof.records.push_back(r);
  }
  g_prof.enabled = true;
  return 0;
}

int nblahip_profile_reset(void) {
  std::lock_guard<std::mutex> lock(g_prof.mu);
  g_prof.used = 0;
  g_prof.dropped = 0;
  return 0;
}

int nblahip_profile_query(const char *kernel_name, double *total_ms, int64_t *launches) {
  if (!kernel_name || !total_ms || !launches) return NBLAHIP_EINVAL;
  std::lock_guard<std::mutex> lock(g_prof.mu);
  *total_ms = 0.0;
  *launches = 0;
  for (size_t i = 0; i < g_prof.used; ++i) {
    const ProfRecord &r = g_prof.records[i];
    if (std::strcmp(r.tag, kernel_name) != 0) continue;
    hipError_t e = hipEventSynchronize(r.stop);
    if (e != hipSuccess) return static_cast<int>(e);
    float ms = 0.f;
    e = hipEventElapsedTime(&ms, r.start, r.stop);
    if (e != hipSuccess) return static_cast<int>(e);
    *total_ms += ms;
    *launches += 1;
  }
  return 0;
}

int nblahip_profile_kernels(char *names, size_t capacity, size_t *needed) {
  if (!needed || (!names && capacity)) return NBLAHIP_EINVAL;
  std::lock_guard<std::mutex> lock(g_prof.mu);
  std::vector<const char *> seen;
  std::string out;
  for (size_t i = 0; i < g_prof.used; ++i) {
    const char *tag = g_prof.records[i].tag;
    bool dup = false;
    for (const char *t : seen) dup = dup || std::strcmp(t, tag) == 0;
    if (dup) continue;
    seen.push_back(tag);
    if (!out.empty()) out += '\n';
    out += tag;
  }
  *needed = out.size() + 1;
  if (capacity) {
    const size_t n = out.size() < capacity - 1 ? out.size() : capacity - 1;
    std::memcpy(names, out.data(), n);
    names[n] = '\0';
  }
  return 0;
}

int nblahip_tune_set(const char *name, int value) {
  if (!name || !*name || value >= (1 << 20)) return NBLAHIP_EINVAL;
  std::lock_guard<std::mutex> lock(g_tune_mu);
  tune_entry_locked(name).set = value < 0 ? -1 : value;
  return 0;
}

int nblahip_tune_get(const char *name, int fallback) {
  if (!name || !*name) return fallback;
  return tune_int(name, fallback);
}

int nblahip_tune_reset(void) {
  std::lock_guard<std::mutex> lock(g_tune_mu);
  for (auto &kv : g_tune) kv.second.set = -1;
  return 0;
}

int nblahip_device_count(int *count) {
  if (!count) return NBLAHIP_EINVAL;
  return hip_status(hipGetDeviceCount(count));
}
int nblahip_set_device(int device) { return hip_status(hipSetDevice(device)); }
int nblahip_get_device(int *device) {
  if (!device) return NBLAHIP_EINVAL;
  return hip_status(hipGetDevice(device));
}
int nblahip_device_synchronize(void) { return hip_status(hipDeviceSynchronize()); }
int nblahip_stream_synchronize(void *stream) {
  return hip_status(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

int nblahip_device_info(int device, char *name, size_t name_len, int *compute_units,
                        int *wave_size, size_t *total_mem) {
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return static_cast<int>(e);
  if (name && name_len) {
    std::strncpy(name, prop.name, name_len - 1);
    name[name_len - 1] = '\0';
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (wave_size) *wave_size = prop.warpSize;
  if (total_mem) *total_mem = prop.totalGlobalMem;
  return 0;
}

int nblahip_malloc(void **ptr, size_t bytes) {
  if (!ptr) return NBLAHIP_EINVAL;
  *ptr = nullptr;
  if (bytes == 0) return 0;
  return hip_status(hipMalloc(ptr, bytes));
}
int nblahip_free(void *ptr) { return ptr ? hip_status(hipFree(ptr)) : 0; }

int nblahip_host_malloc(void **ptr, size_t bytes) {
  if (!ptr) return NBLAHIP_EINVAL;
  *ptr = nullptr;
  if (bytes == 0) return 0;
  return hip_status(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
}
int nblahip_host_free(void *ptr) { return ptr ? hip_status(hipHostFree(ptr)) : 0; }

int nblahip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return NBLAHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int e = hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, st))) return e;
  return hip_status(hipStreamSynchronize(st)); // pageable host memory: make the call blocking
}
int nblahip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return NBLAHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int e = hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, st))) return e;
  return hip_status(hipStreamSynchronize(st));
}
// Non-blocking copies for page-locked host memory: enqueued on `stream`, the
// caller orders them with events.
int nblahip_memcpy_h2d_async(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return NBLAHIP_EINVAL;
  return hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
                                   static_cast<hipStream_t>(stream)));
}
int nblahip_memcpy_d2h_async(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return NBLAHIP_EINVAL;
  return hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
                                   static_cast<hipStream_t>(stream)));
}

int nblahip_stream_create(void **stream) {
  if (!stream) return NBLAHIP_EINVAL;
  hipStream_t st = nullptr;
  // default priority; non-blocking: ordered against the null stream by events only
  const int e = hip_status(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  *stream = st;
  return e;
}
int nblahip_stream_destroy(void *stream) {
  return stream ? hip_status(hipStreamDestroy(static_cast<hipStream_t>(stream))) : 0;
}
int nblahip_event_create(void **event) {
  if (!event) return NBLAHIP_EINVAL;
  hipEvent_t ev = nullptr;
  const int e = hip_status(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  *event = ev;
  return e;
}
int nblahip_event_destroy(void *event) {
  return event ? hip_status(hipEventDestroy(static_cast<hipEvent_t>(event))) : 0;
}
int nblahip_event_record(void *event, void *stream) {
  if (!event) return NBLAHIP_EINVAL;
  return hip_status(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}
int nblahip_stream_wait_event(void *stream, void *event) {
  if (!event) return NBLAHIP_EINVAL;
  return hip_status(hipStreamWaitEvent(static_cast<hipStream_t>(stream),
                                       static_cast<hipEvent_t>(event), 0));
}
int nblahip_event_synchronize(void *event) {
  if (!event) return NBLAHIP_EINVAL;
  return hip_status(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}
int nblahip_event_query(void *event, int *done) {
  if (!event || !done) return NBLAHIP_EINVAL;
  const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipErrorNotReady) {
    *done = 0;
    return 0;
  }
  *done = e == hipSuccess ? 1 : 0;
  return hip_status(e);
}

int nblahip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return NBLAHIP_EINVAL;
  return hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice,
                                   static_cast<hipStream_t>(stream)));
}
int nblahip_memset(void *dst, int byte, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (!dst) return NBLAHIP_EINVAL;
  return hip_status(hipMemsetAsync(dst, byte, bytes, static_cast<hipStream_t>(stream)));
}

int nblahip_convert(void *dst, int dst_dtype, const void *src, int src_dtype, int64_t n,
                    void *stream) {
  if (n == 0) return 0;
  if (!dst || !src || n < 0) return NBLAHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g(flat_grid(n)), b(256);
  if (dst_dtype == NBLAHIP_F32 && src_dtype == NBLAHIP_F16) {
    NBLAHIP_LAUNCH("convert_kernel", (convert_kernel<float, __half>), g, b, 0, st, static_cast<float *>(dst),
                       static_cast<const __half *>(src), n);
  } else if (dst_dtype == NBLAHIP_F16 && src_dtype == NBLAHIP_F32) {
    NBLAHIP_LAUNCH("convert_kernel", (convert_kernel<__half, float>), g, b, 0, st, static_cast<__half *>(dst),
                       static_cast<const float *>(src), n);
  } else if (dst_dtype == src_dtype && (dst_dtype == NBLAHIP_F32 || dst_dtype == NBLAHIP_F16)) {
    const size_t bytes = static_cast<size_t>(n) * (dst_dtype == NBLAHIP_F32 ? 4 : 2);
    return hip_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, st));
  } else {
    return NBLAHIP_EINVAL;
  }
  return last_launch_status();
}

int nblahip_fill(void *dst, int dtype, float value, int64_t n, void *stream) {
  if (n == 0) return 0;
  if (!dst || n < 0) return NBLAHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g(flat_grid(n)), b(256);
  if (dtype == NBLAHIP_F32) {
    NBLAHIP_LAUNCH("fill_kernel", (fill_kernel<float>), g, b, 0, st, static_cast<float *>(dst), value, n);
  } else if (dtype == NBLAHIP_F16) {
    NBLAHIP_LAUNCH("fill_kernel", (fill_kernel<__half>), g, b, 0, st, static_cast<__half *>(dst), value, n);
  } else {
    return NBLAHIP_EINVAL;
  }
  return last_launch_status();
}

int nblahip_fill_bytes(void *dst, int elem_bytes, unsigned long long pattern, int64_t n,
                       void *stream) {
  if (n == 0) return 0;
  if (!dst || n < 0) return NBLAHIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(dst) % static_cast<uintptr_t>(elem_bytes > 0 ? elem_bytes : 1))
    return NBLAHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g(flat_grid(n)), b(256);
  switch (elem_bytes) {
  case 1:
    NBLAHIP_LAUNCH("fill_kernel", (fill_words_kernel<uint8_t>), g, b, 0, st, static_cast<uint8_t *>(dst),
                   static_cast<uint8_t>(pattern), n);
    break;
  case 2:
    NBLAHIP_LAUNCH("fill_kernel", (fill_words_kernel<uint16_t>), g, b, 0, st, static_cast<uint16_t *>(dst),
                   static_cast<uint16_t>(pattern), n);
    break;
  case 4:
    NBLAHIP_LAUNCH("fill_kernel", (fill_words_kernel<uint32_t>), g, b, 0, st, static_cast<uint32_t *>(dst),
                   static_cast<uint32_t>(pattern), n);
    break;
  case 8:
    NBLAHIP_LAUNCH("fill_kernel", (fill_words_kernel<unsigned long long>), g, b, 0, st,
                   static_cast<unsigned long long *>(dst), pattern, n);
    break;
  default:
    return NBLAHIP_EINVAL;
  }
  return last_launch_status();
}

int nblahip_stage_params(int count, const void *const *src, int src_dtype, void *const *dst,
                         int dst_dtype, const int64_t *n, void *stream) {
  if (count == 0) return 0;
  if (count < 0 || count > kStageMax || !src || !dst || !n) return NBLAHIP_EINVAL;
  const bool up = src_dtype == NBLAHIP_F16 && dst_dtype == NBLAHIP_F32;
  const bool down = src_dtype == NBLAHIP_F32 && dst_dtype == NBLAHIP_F16;
  if (!up && !down) return NBLAHIP_EINVAL;
  StageArgs a{};
  int64_t longest = 0;
  int used = 0;
  for (int k = 0; k < count; ++k) {
    if (n[k] < 0) return NBLAHIP_EINVAL;
    if (n[k] == 0) continue;
    if (!src[k] || !dst[k]) return NBLAHIP_EINVAL;
    a.src[used] = src[k];
    a.dst[used] = dst[k];
    a.n[used] = n[k];
    longest = std::max(longest, n[k]);
    ++used;
  }
  if (used == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g(std::min(flat_grid(longest), 1024u), used), b(256);
  if (up) {
    NBLAHIP_LAUNCH("stage_params_kernel", (stage_params_kernel<float, __half>), g, b, 0, st, a);
  } else {
    NBLAHIP_LAUNCH("stage_params_kernel", (stage_params_kernel<__half, float>), g, b, 0, st, a);
  }
  return last_launch_status();
}

int nblahip_xchg_set_epoch(unsigned int epoch) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return hip_status(e);
  xchg_debug_set_epoch(dev, epoch);
  return 0;
}

} // extern "C"
