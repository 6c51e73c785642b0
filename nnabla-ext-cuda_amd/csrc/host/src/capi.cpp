// Flat C surface over the C++ backend (see include/nnabla_hip_capi.h).
#include <cstring>
#include <nnabla_hip_capi.h>

#include <nbla/cpu.hpp>
#include <nbla/function/batch_normalization.hpp>
#include <nbla/function/fused_batch_normalization.hpp>
#include <nbla/function/group_normalization.hpp>
#include <nbla/function/instance_normalization.hpp>
#include <nbla/function/layer_normalization.hpp>
#include <nbla/function/tensor_normalization.hpp>
#include <nbla/function/weight_standardization.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/init.hpp>
#include <nbla/variable.hpp>

using namespace nbla;

struct nnabla_hip_variable {
  Variable var;
  explicit nnabla_hip_variable(const Shape_t &s) : var(s) {}
};
struct nnabla_hip_function {
  FunctionPtr fn;
  string name;
};

namespace {
thread_local string g_last_error;

template <typename F> int guarded(F &&f) {
  try {
    f();
    return 0;
  } catch (const Exception &e) {
    g_last_error = e.what();
    return 1 + static_cast<int>(e.code());
  } catch (const std::exception &e) {
    g_last_error = e.what();
    return 100;
  } catch (...) {
    g_last_error = "unknown exception";
    return 101;
  }
}

vector<string> split(const char *s) {
  vector<string> out;
  string cur;
  for (const char *p = s ? s : ""; *p; ++p) {
    if (*p == ',') {
      if (!cur.empty()) out.push_back(cur);
      cur.clear();
    } else if (*p != ' ') {
      cur.push_back(*p);
    }
  }
  if (!cur.empty()) out.push_back(cur);
  return out;
}

Context make_ctx(const char *backends, const char *array_class, const char *device_id) {
  return Context(split(backends), array_class ? array_class : "HipCachedArray",
                 device_id ? device_id : "0");
}

Variables to_vars(nnabla_hip_variable **v, int n) {
  Variables out;
  for (int i = 0; i < n; ++i) {
    NBLA_CHECK(v && v[i], error_code::value, "null variable handle at position %d", i);
    out.push_back(&v[i]->var);
  }
  return out;
}

NdArrayPtr pick(nnabla_hip_variable *v, int which) {
  NBLA_CHECK(v, error_code::value, "null variable handle");
  NBLA_CHECK(which == 0 || which == 1, error_code::value, "which must be 0 (data) or 1 (grad)");
  return which == 0 ? v->var.data() : v->var.grad();
}

// Array class the host side of variable_set/get stages through.
std::string &host_array_class() {
  static std::string name = "CpuArray";
  return name;
}

Context host_ctx() { return Context({"cpu:float"}, host_array_class(), "0"); }

nnabla_hip_function *wrap(FunctionPtr fn) {
  nnabla_hip_function *f = new nnabla_hip_function;
  f->fn = fn;
  f->name = fn->name();
  return f;
}
} // namespace

extern "C" {

int nnabla_hip_init(void) {
  return guarded([] { init_hip(); });
}

const char *nnabla_hip_last_error(void) { return g_last_error.c_str(); }

const char *nnabla_hip_array_classes(void) {
  static string joined;
  joined.clear();
  for (const string &s : SingletonManager::get<Hip>()->array_classes())
    joined += (joined.empty() ? "" : ",") + s;
  return joined.c_str();
}

int nnabla_hip_device_synchronize(const char *device_id) {
  return guarded([&] { SingletonManager::get<Hip>()->device_synchronize(device_id ? device_id : "0"); });
}

int nnabla_hip_memory_stats(uint64_t *live_bytes, uint64_t *cached_bytes) {
  return guarded([&] {
    if (live_bytes) *live_bytes = SingletonManager::get<Hip>()->live_bytes();
    if (cached_bytes) *cached_bytes = SingletonManager::get<Hip>()->cached_bytes();
  });
}

int nnabla_hip_clear_memory_cache(void) {
  return guarded([] { SingletonManager::get<Hip>()->free_unused_device_caches(); });
}

nnabla_hip_variable *nnabla_hip_variable_new(int ndim, const int64_t *shape) {
  nnabla_hip_variable *out = nullptr;
  guarded([&] {
    NBLA_CHECK(ndim >= 0 && (ndim == 0 || shape), error_code::value, "bad shape");
    Shape_t s(shape, shape + ndim);
    for (Size_t d : s) NBLA_CHECK(d >= 0, error_code::value, "negative dimension");
    out = new nnabla_hip_variable(s);
  });
  return out;
}

void nnabla_hip_variable_delete(nnabla_hip_variable *v) { delete v; }

int nnabla_hip_variable_ndim(nnabla_hip_variable *v) { return v ? static_cast<int>(v->var.ndim()) : -1; }

int nnabla_hip_variable_shape(nnabla_hip_variable *v, int64_t *shape_out) {
  return guarded([&] {
    NBLA_CHECK(v && shape_out, error_code::value, "null argument");
    const Shape_t s = v->var.shape();
    std::copy(s.begin(), s.end(), shape_out);
  });
}

int nnabla_hip_device_count(int *count) {
  return guarded([&] {
    NBLA_CHECK(count, error_code::value, "count must not be null");
    NBLA_HIP_CHECK(nblahip_device_count(count));
  });
}

int nnabla_hip_set_host_array_class(const char *name) {
  return guarded([&] {
    const std::string n = name ? name : "";
    NBLA_CHECK(n == "CpuArray" || n == "HipCachedHostArray", error_code::value,
               "host array class must be CpuArray or HipCachedHostArray, given '%s'", n.c_str());
    if (n != "CpuArray") init_hip();
    host_array_class() = n;
  });
}

int nnabla_hip_variable_set(nnabla_hip_variable *v, int which, const float *host, int64_t n,
                            int dtype) {
  return guarded([&] {
    NdArrayPtr a = pick(v, which);
    NBLA_CHECK(host && n == a->size(), error_code::value, "expected %lld elements, given %lld",
               static_cast<long long>(a->size()), static_cast<long long>(n));
    NBLA_CHECK(dtype == 0 || dtype == 1, error_code::value, "dtype must be 0 (float) or 1 (half)");
    init_cpu();
    if (dtype == 0) {
      float *dst = a->cast(dtypes::FLOAT, host_ctx(), true)->pointer<float>();
      std::copy(host, host + n, dst);
    } else {
      Half *dst = a->cast(dtypes::HALF, host_ctx(), true)->pointer<Half>();
      for (int64_t i = 0; i < n; ++i) dst[i] = Half(host[i]);
    }
  });
}

int nnabla_hip_variable_get(nnabla_hip_variable *v, int which, float *host, int64_t n) {
  return guarded([&] {
    NdArrayPtr a = pick(v, which);
    NBLA_CHECK(host && n == a->size(), error_code::value, "expected %lld elements, given %lld",
               static_cast<long long>(a->size()), static_cast<long long>(n));
    init_cpu();
    const float *src = a->get(dtypes::FLOAT, host_ctx())->const_pointer<float>();
    std::copy(src, src + n, host);
  });
}

namespace {
// 0: float, 1: half, 0x100 + n: the core's dtypes enumerator n (any stored type).
dtypes storage_dtype(int dtype) {
  if (dtype == 0) return dtypes::FLOAT;
  if (dtype == 1) return dtypes::HALF;
  const int n = dtype - 0x100;
  NBLA_CHECK((n >= static_cast<int>(dtypes::BOOL) && n <= static_cast<int>(dtypes::DOUBLE)) ||
                 n == static_cast<int>(dtypes::HALF),
             error_code::value, "dtype must be 0 (float), 1 (half) or 0x100 + a core dtype");
  return static_cast<dtypes>(n);
}
} // namespace

int nnabla_hip_variable_cast(nnabla_hip_variable *v, int which, const char *array_class,
                             const char *device_id, int dtype, int write_only, int async_flags) {
  return guarded([&] {
    NdArrayPtr a = pick(v, which);
    NBLA_CHECK(array_class != nullptr, error_code::value, "array_class must be given");
    init_hip();
    const Context ctx({}, array_class, device_id ? device_id : "0");
    a->cast(storage_dtype(dtype), ctx, write_only != 0, async_flags);
  });
}

int nnabla_hip_variable_set_raw(nnabla_hip_variable *v, int which, const void *host, int64_t n,
                                int dtype) {
  return guarded([&] {
    NdArrayPtr a = pick(v, which);
    NBLA_CHECK(host && n == a->size(), error_code::value, "expected %lld elements, given %lld",
               static_cast<long long>(a->size()), static_cast<long long>(n));
    init_cpu();
    const dtypes d = storage_dtype(dtype);
    void *dst = a->cast(d, host_ctx(), true)->pointer<void>();
    std::memcpy(dst, host, static_cast<size_t>(n) * sizeof_dtype(d));
  });
}

int nnabla_hip_variable_get_raw(nnabla_hip_variable *v, int which, void *host, int64_t n,
                                int dtype) {
  return guarded([&] {
    NdArrayPtr a = pick(v, which);
    NBLA_CHECK(host && n == a->size(), error_code::value, "expected %lld elements, given %lld",
               static_cast<long long>(a->size()), static_cast<long long>(n));
    init_cpu();
    const dtypes d = storage_dtype(dtype);
    const void *src = a->get(d, host_ctx())->const_pointer<void>();
    std::memcpy(host, src, static_cast<size_t>(n) * sizeof_dtype(d));
  });
}

int nnabla_hip_pending_transfers(uint64_t *count) {
  return guarded([&] {
    NBLA_CHECK(count != nullptr, error_code::value, "count must not be null");
    *count = SingletonManager::get<Hip>()->pending_transfers();
  });
}

int nnabla_hip_variable_zero(nnabla_hip_variable *v, int which) {
  return guarded([&] { pick(v, which)->zero(); });
}

int nnabla_hip_variable_fill(nnabla_hip_variable *v, int which, float value) {
  return guarded([&] { pick(v, which)->fill(value); });
}

int nnabla_hip_variable_stored_dtype(nnabla_hip_variable *v, int which, int *dtype) {
  return guarded([&] {
    NBLA_CHECK(dtype, error_code::value, "dtype is null");
    NdArrayPtr a = pick(v, which);
    try {
      const dtypes d = a->array()->dtype();
      *dtype = d == dtypes::FLOAT ? 0 : d == dtypes::HALF ? 1 : 0x100 + static_cast<int>(d);
    } catch (...) {
      *dtype = -1;
    }
  });
}

nnabla_hip_function *nnabla_hip_create_batch_normalization(const char *backends,
                                                           const char *array_class,
                                                           const char *device_id, const int *axes,
                                                           int n_axes, float decay_rate, float eps,
                                                           int batch_stat, int no_scale,
                                                           int no_bias) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ax(axes, axes + n_axes);
    out = wrap(create_BatchNormalization(make_ctx(backends, array_class, device_id), ax, decay_rate,
                                         eps, batch_stat != 0, no_scale != 0, no_bias != 0));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_fused_batch_normalization(
    const char *backends, const char *array_class, const char *device_id, const int *axes,
    int n_axes, float decay_rate, float eps, int batch_stat, const char *nonlinearity) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ax(axes, axes + n_axes);
    out = wrap(create_FusedBatchNormalization(make_ctx(backends, array_class, device_id), ax,
                                              decay_rate, eps, batch_stat != 0,
                                              string(nonlinearity ? nonlinearity : "")));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_layer_normalization(const char *backends,
                                                           const char *array_class,
                                                           const char *device_id,
                                                           const int *batch_axis, int n_batch_axis,
                                                           float eps, int no_scale, int no_bias) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ba(batch_axis, batch_axis + n_batch_axis);
    out = wrap(create_LayerNormalization(make_ctx(backends, array_class, device_id), ba, eps,
                                         no_scale != 0, no_bias != 0));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_group_normalization(const char *backends,
                                                           const char *array_class,
                                                           const char *device_id, int num_groups,
                                                           int channel_axis, const int *batch_axis,
                                                           int n_batch_axis, float eps, int no_scale,
                                                           int no_bias) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ba(batch_axis, batch_axis + n_batch_axis);
    out = wrap(create_GroupNormalization(make_ctx(backends, array_class, device_id), num_groups,
                                         channel_axis, ba, eps, no_scale != 0, no_bias != 0));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_instance_normalization(const char *backends,
                                                              const char *array_class,
                                                              const char *device_id,
                                                              int channel_axis,
                                                              const int *batch_axis,
                                                              int n_batch_axis, float eps,
                                                              int no_scale, int no_bias) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ba(batch_axis, batch_axis + n_batch_axis);
    out = wrap(create_InstanceNormalization(make_ctx(backends, array_class, device_id),
                                            channel_axis, ba, eps, no_scale != 0, no_bias != 0));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_tensor_normalization(const char *backends,
                                                            const char *array_class,
                                                            const char *device_id, const int *axes,
                                                            int n_axes, float eps, int no_scale,
                                                            int no_bias) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    const vector<int> ax(axes, axes + n_axes);
    out = wrap(create_TensorNormalization(make_ctx(backends, array_class, device_id), ax, eps,
                                          no_scale != 0, no_bias != 0));
  });
  return out;
}

nnabla_hip_function *nnabla_hip_create_weight_standardization(const char *backends,
                                                              const char *array_class,
                                                              const char *device_id,
                                                              int channel_axis, float eps) {
  nnabla_hip_function *out = nullptr;
  guarded([&] {
    out = wrap(create_WeightStandardization(make_ctx(backends, array_class, device_id),
                                            channel_axis, eps));
  });
  return out;
}

void nnabla_hip_function_delete(nnabla_hip_function *f) { delete f; }

const char *nnabla_hip_function_name(nnabla_hip_function *f) { return f ? f->name.c_str() : ""; }

int nnabla_hip_function_setup(nnabla_hip_function *f, nnabla_hip_variable **inputs, int n_inputs,
                              nnabla_hip_variable **outputs, int n_outputs) {
  return guarded([&] {
    NBLA_CHECK(f, error_code::value, "null function handle");
    f->fn->setup(to_vars(inputs, n_inputs), to_vars(outputs, n_outputs));
  });
}

int nnabla_hip_function_forward(nnabla_hip_function *f, nnabla_hip_variable **inputs, int n_inputs,
                                nnabla_hip_variable **outputs, int n_outputs) {
  return guarded([&] {
    NBLA_CHECK(f, error_code::value, "null function handle");
    f->fn->forward(to_vars(inputs, n_inputs), to_vars(outputs, n_outputs));
  });
}

int nnabla_hip_function_recompute(nnabla_hip_function *f, nnabla_hip_variable **inputs,
                                  int n_inputs, nnabla_hip_variable **outputs, int n_outputs) {
  return guarded([&] {
    NBLA_CHECK(f, error_code::value, "null function handle");
    f->fn->recompute(to_vars(inputs, n_inputs), to_vars(outputs, n_outputs));
  });
}

int nnabla_hip_function_backward(nnabla_hip_function *f, nnabla_hip_variable **inputs, int n_inputs,
                                 nnabla_hip_variable **outputs, int n_outputs,
                                 const int *propagate_down, const int *accum) {
  return guarded([&] {
    NBLA_CHECK(f && propagate_down && accum, error_code::value, "null argument");
    vector<bool> pd(n_inputs), ac(n_inputs);
    for (int i = 0; i < n_inputs; ++i) {
      pd[i] = propagate_down[i] != 0;
      ac[i] = accum[i] != 0;
    }
    f->fn->backward(to_vars(inputs, n_inputs), to_vars(outputs, n_outputs), pd, ac);
  });
}

} // extern "C"
