// Minimal stand-in for the NNabla core (sony/nnabla), which is not part of the
// extension tree the backend is modelled on.  It provides exactly the types the
// normalization Function classes touch, with the semantics read off the
// reference's call sites (cited per type):
//   Context, Shape_t/Size_t, dtypes, Half, Exception + NBLA_CHECK/NBLA_ERROR,
//   Array / ArrayCreator / ArraySynchronizer, SyncedArray, NdArray, Variable,
//   Function (setup/forward/backward/recompute, fall_back_func_),
//   FunctionRegistry + NBLA_REGISTER_FUNCTION_* macros, SingletonManager,
//   BackendBase/BackendUtils.
// When a real libnnabla is on the include path (nbla/function.hpp exists ahead
// of this directory) its headers are used instead and this file is never seen.
//
// There is deliberately NO CPU implementation of any normalization here: a
// context that lists only "cpu:float" finds no registered implementation and
// raises.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <memory>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <string>
#include <tuple>
#include <typeindex>
#include <unordered_map>
#include <utility>
#include <vector>

#define NBLA_API __attribute__((visibility("default")))

namespace nbla {

using std::make_shared;
using std::shared_ptr;
using std::string;
using std::vector;

// ---------------------------------------------------------------- errors
// (NBLA_ERROR / NBLA_CHECK and error_code as used at
// include/nbla/cuda/common.hpp:70-85.)
enum class error_code {
  unclassified = 0,
  not_implemented,
  value,
  type,
  memory,
  io,
  os,
  target_specific,
  target_specific_async,
  runtime
};

inline const char *get_error_string(error_code c) {
  switch (c) {
  case error_code::not_implemented: return "NotImplementedError";
  case error_code::value: return "ValueError";
  case error_code::type: return "TypeError";
  case error_code::memory: return "MemoryError";
  case error_code::io: return "IOError";
  case error_code::os: return "OSError";
  case error_code::target_specific: return "TargetSpecificError";
  case error_code::target_specific_async: return "TargetSpecificAsyncError";
  case error_code::runtime: return "RuntimeError";
  default: return "UnclassifiedError";
  }
}

class NBLA_API Exception : public std::exception {
  error_code code_;
  string full_msg_;

public:
  Exception(error_code code, const string &msg, const string &func, const string &file, int line)
      : code_(code) {
    std::ostringstream ss;
    ss << get_error_string(code) << " in " << func << "\n" << file << ":" << line << "\n" << msg;
    full_msg_ = ss.str();
  }
  const char *what() const noexcept override { return full_msg_.c_str(); }
  error_code code() const { return code_; }
};

inline string format_string(const char *fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  return string(buf);
}
inline string format_string() { return string(); }

#define NBLA_ERROR(code, ...)                                                          \
  throw ::nbla::Exception(code, ::nbla::format_string(__VA_ARGS__), __func__, __FILE__, __LINE__)

#define NBLA_CHECK(condition, code, ...)                                               \
  do {                                                                                 \
    if (!(condition)) {                                                                \
      throw ::nbla::Exception(code,                                                    \
                              ::nbla::string("Failed `" #condition "`: ") +            \
                                  ::nbla::format_string(__VA_ARGS__),                  \
                              __func__, __FILE__, __LINE__);                           \
    }                                                                                  \
  } while (0)

// ---------------------------------------------------------------- basics
typedef int64_t Size_t;
typedef vector<Size_t> Shape_t;

// (dtypes::FLOAT / HALF and sizeof_dtype as used at
// src/nbla/cuda/cudnn/function/generic/batch_normalization.cu:363,374.)
enum class dtypes { BOOL = 0, BYTE, UBYTE, SHORT, USHORT, INT, UINT, LONG, ULONG, FLOAT, DOUBLE, HALF = 23 };

inline size_t sizeof_dtype(dtypes d) {
  switch (d) {
  case dtypes::BOOL: case dtypes::BYTE: case dtypes::UBYTE: return 1;
  case dtypes::SHORT: case dtypes::USHORT: case dtypes::HALF: return 2;
  case dtypes::INT: case dtypes::UINT: case dtypes::FLOAT: return 4;
  default: return 8;
  }
}

// 16-bit float storage type (include/nbla/cuda/half.hpp:55-70 wraps `.bits`).
struct Half {
  uint16_t bits;
  Half() : bits(0) {}
  Half(float f) { bits = from_float(f); }
  operator float() const { return to_float(bits); }
  static uint16_t from_float(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const int32_t exp = static_cast<int32_t>((x >> 23) & 0xff) - 127 + 15;
    uint32_t mant = x & 0x7fffffu;
    if (((x >> 23) & 0xff) == 0xff) return static_cast<uint16_t>(sign | 0x7c00u | (mant ? 0x200u : 0));
    if (exp >= 31) return static_cast<uint16_t>(sign | 0x7c00u);
    if (exp <= 0) {
      if (exp < -10) return static_cast<uint16_t>(sign);
      mant |= 0x800000u;
      const int shift = 14 - exp;
      uint32_t h = mant >> shift;
      const uint32_t rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
      if (rem > half || (rem == half && (h & 1))) ++h;
      return static_cast<uint16_t>(sign | h);
    }
    uint32_t h = (static_cast<uint32_t>(exp) << 10) | (mant >> 13);
    const uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
    return static_cast<uint16_t>(sign | h);
  }
  static float to_float(uint16_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, x;
    if (exp == 0) {
      if (mant == 0) {
        x = sign;
      } else {
        int e = -1;
        do { ++e; mant <<= 1; } while (!(mant & 0x400u));
        x = sign | (static_cast<uint32_t>(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
      }
    } else if (exp == 31) {
      x = sign | 0x7f800000u | (mant << 13);
    } else {
      x = sign | ((exp + 127 - 15) << 23) | (mant << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
  }
};

template <typename T> inline dtypes get_dtype();
template <> inline dtypes get_dtype<float>() { return dtypes::FLOAT; }
template <> inline dtypes get_dtype<Half>() { return dtypes::HALF; }
template <> inline dtypes get_dtype<int>() { return dtypes::INT; }
template <> inline dtypes get_dtype<char>() { return dtypes::BYTE; }

inline Size_t compute_size_by_shape(const Shape_t &shape, Size_t axis = 0) {
  Size_t s = 1;
  for (size_t i = static_cast<size_t>(axis); i < shape.size(); ++i) s *= shape[i];
  return s;
}

// (Context{backend list, array class, device id} as built at
// examples/cpp/mnist_training/main.cpp:42-43.)
struct Context {
  vector<string> backend;
  string array_class;
  string device_id;
  Context(const vector<string> &b = {"cpu:float"}, const string &a = "CpuArray",
          const string &d = "0")
      : backend(b), array_class(a), device_id(d) {}
  string to_string() const {
    string s = "Context(backend=[";
    for (size_t i = 0; i < backend.size(); ++i) s += (i ? "," : "") + backend[i];
    return s + "], array_class=" + array_class + ", device_id=" + device_id + ")";
  }
};

// ---------------------------------------------------------------- singleton
class NBLA_API SingletonManager {
public:
  template <typename S> static S *get() {
    static S *instance = new S(); // intentionally leaked: lives to process end
    return instance;
  }
};

// ---------------------------------------------------------------- arrays
// Flags of a cast / get / synchronizer call (used as AsyncFlag::ASYNC etc. at
// src/nbla/cuda/array/cuda_array.cpp:130,149,191,199): ASYNC asks for a
// non-blocking transfer, UNSAFE waives keeping the source alive until the
// transfer has run, OFFREC belongs to the core's array-use recorder.
namespace AsyncFlag {
enum Flags { NONE = 0, ASYNC = 1, UNSAFE = 2, OFFREC = 4 };
}

inline bool is_cpu_context(const Context &ctx) {
  return ctx.array_class.find("Cpu") == 0 || ctx.array_class.find("HostArray") != string::npos;
}

// An asynchronous transfer still on its way into an array
// (include/nbla/cuda/event.hpp: CudaEvent derives from this).
class NBLA_API Event {
public:
  virtual ~Event() {}
  // Makes the consumer (the function stream, and the host for a host
  // consumer without ASYNC / UNSAFE) wait for the transfer.
  virtual void wait_event(const Context ctx, const int async_flags = AsyncFlag::NONE) = 0;
};
typedef shared_ptr<Event> EventPtr;

// (Array interface as subclassed at include/nbla/cuda/array/cuda_array.hpp:36-49.)
class NBLA_API Array : public std::enable_shared_from_this<Array> {
protected:
  Size_t size_;
  dtypes dtype_;
  Context ctx_;
  void *ptr_ = nullptr;
  EventPtr event_;

public:
  Array(Size_t size, dtypes dtype, const Context &ctx) : size_(size), dtype_(dtype), ctx_(ctx) {}
  virtual ~Array() {}
  shared_ptr<Array> getptr() { return shared_from_this(); }
  // The transfer that fills this array, if one is still outstanding
  // (cuda_array.cpp:87-91,113-114: set by the asynchronous synchronizers,
  // consumed by wait_event).
  void set_event(EventPtr e) { event_ = e; }
  bool have_event() const { return static_cast<bool>(event_); }
  void wait_event(const Context ctx, const int async_flags = AsyncFlag::NONE) {
    if (event_) {
      event_->wait_event(ctx, async_flags);
      event_.reset();
    }
  }
  template <typename T = void> T *pointer() { return reinterpret_cast<T *>(ptr_); }
  template <typename T = void> const T *const_pointer() const {
    return reinterpret_cast<const T *>(ptr_);
  }
  Size_t size() const { return size_; }
  dtypes dtype() const { return dtype_; }
  const Context &context() const { return ctx_; }
  size_t nbytes() const { return static_cast<size_t>(size_) * sizeof_dtype(dtype_); }
  virtual void zero() = 0;
  virtual void fill(float value) = 0;
  // Same array class, possibly different dtype.
  virtual void copy_from(const Array *src) = 0;
};
typedef shared_ptr<Array> ArrayPtr;

// (NBLA_REGISTER_ARRAY_CREATOR / _SYNCHRONIZER at src/nbla/cuda/init.cpp.tmpl:93-220.)
class NBLA_API ArrayCreator {
public:
  typedef std::function<Array *(Size_t, dtypes, const Context &)> Creator;
  static std::map<string, Creator> &registry() {
    static std::map<string, Creator> r;
    return r;
  }
  static void add_creator(const string &name, Creator c) { registry()[name] = c; }
  static Array *create(Size_t size, dtypes dtype, const Context &ctx) {
    auto it = registry().find(ctx.array_class);
    NBLA_CHECK(it != registry().end(), error_code::unclassified, "Array class '%s' is not registered.",
               ctx.array_class.c_str());
    return it->second(size, dtype, ctx);
  }
};

class NBLA_API ArraySynchronizer {
public:
  typedef std::function<void(Array *, Array *, const int)> Synchronizer; // (src, dst, async_flags)
  static std::map<std::pair<string, string>, Synchronizer> &registry() {
    static std::map<std::pair<string, string>, Synchronizer> r;
    return r;
  }
  static void add_synchronizer(const string &src, const string &dst, Synchronizer s) {
    registry()[std::make_pair(src, dst)] = s;
  }
  static void synchronize(const string &src_class, Array *src, const string &dst_class, Array *dst,
                          const int async_flags = AsyncFlag::NONE) {
    auto it = registry().find(std::make_pair(src_class, dst_class));
    NBLA_CHECK(it != registry().end(), error_code::unclassified,
               "No synchronizer registered from %s to %s.", src_class.c_str(), dst_class.c_str());
    it->second(src, dst, async_flags);
  }
};

// Host array (the core's CpuArray, minimal).
class NBLA_API CpuArray : public Array {
protected:
  bool owns_ = true;
  // For subclasses that bring their own host storage (the core passes an
  // AllocatorMemoryPtr: src/nbla/cuda/array/cuda_array.cpp:283-296).
  CpuArray(Size_t size, dtypes dtype, const Context &ctx, void *storage)
      : Array(size, dtype, ctx), owns_(false) {
    ptr_ = storage;
  }

public:
  CpuArray(Size_t size, dtypes dtype, const Context &ctx) : Array(size, dtype, ctx) {
    ptr_ = std::malloc(std::max<size_t>(nbytes(), 1));
    NBLA_CHECK(ptr_, error_code::memory, "host allocation of %zu bytes failed", nbytes());
  }
  ~CpuArray() override {
    if (owns_) std::free(ptr_);
  }
  void zero() override { std::memset(ptr_, 0, nbytes()); }
  void fill(float value) override {
    if (dtype_ == dtypes::FLOAT) {
      std::fill_n(pointer<float>(), size_, value);
    } else if (dtype_ == dtypes::HALF) {
      std::fill_n(pointer<Half>(), size_, Half(value));
    } else {
      NBLA_ERROR(error_code::not_implemented, "CpuArray::fill: dtype not supported");
    }
  }
  void copy_from(const Array *src) override {
    NBLA_CHECK(src->size() == size_, error_code::value, "size mismatch");
    if (src->dtype() == dtype_) {
      std::memcpy(ptr_, src->const_pointer<void>(), nbytes());
    } else if (src->dtype() == dtypes::FLOAT && dtype_ == dtypes::HALF) {
      const float *s = src->const_pointer<float>();
      Half *d = pointer<Half>();
      for (Size_t i = 0; i < size_; ++i) d[i] = Half(s[i]);
    } else if (src->dtype() == dtypes::HALF && dtype_ == dtypes::FLOAT) {
      const Half *s = src->const_pointer<Half>();
      float *d = pointer<float>();
      for (Size_t i = 0; i < size_; ++i) d[i] = static_cast<float>(s[i]);
    } else {
      NBLA_ERROR(error_code::not_implemented, "CpuArray::copy_from: dtype pair not supported");
    }
  }
  static Context filter_context(const Context &ctx) { return Context({}, "CpuArray", ""); }
};

// ---------------------------------------------------------------- SyncedArray
// One logical buffer with per-(array class, dtype) materialisations and a head
// that names the up-to-date one.  cast() makes the requested materialisation
// the head (copying unless write_only), get() reads through it.
// (Usage: NdArray::cast(dtype, ctx, write_only)->pointer(), get(dtype, ctx)
// ->const_pointer(), zero(), fill(), array()->clear():
// src/nbla/cuda/function/generic/layer_normalization.cu:91-93,202-203,218.)
class NBLA_API SyncedArray {
  Size_t size_;
  typedef std::pair<string, int> Key; // (array class, dtype)
  std::map<Key, ArrayPtr> arrays_;
  bool has_head_ = false;
  Key head_;
  std::set<Key> current_; // materialisations that hold the head's content (head included)
  bool zeroing_ = false, filling_ = false;
  float fill_value_ = 0.f;

  ArrayPtr materialize(const Key &key, const Context &ctx) {
    auto it = arrays_.find(key);
    if (it != arrays_.end()) return it->second;
    ArrayPtr a(ArrayCreator::create(size_, static_cast<dtypes>(key.second), ctx));
    arrays_[key] = a;
    return a;
  }

  ArrayPtr sync(dtypes dtype, const Context &ctx, bool write_only, const int async_flags) {
    const Key key(ctx.array_class, static_cast<int>(dtype));
    ArrayPtr dst = materialize(key, ctx);
    // A transfer into this materialisation that is still outstanding: its
    // consumer waits here (the function stream; the host too for a host
    // context without ASYNC / UNSAFE).
    dst->wait_event(ctx, async_flags);
    if (write_only) return dst;
    if (!has_head_) {
      // Never written: defined content is zero (or the pending fill value).
      if (filling_) dst->fill(fill_value_); else dst->zero();
      return dst;
    }
    if (zeroing_ || filling_) {
      if (filling_) dst->fill(fill_value_); else dst->zero();
      return dst;
    }
    if (key == head_ || current_.count(key)) return dst; // a reader's copy stays good until the next write
    ArrayPtr src = arrays_.at(head_);
    if (head_.first == key.first) {
      src->wait_event(ctx, async_flags);
      dst->copy_from(src.get()); // same class: dtype conversion on its device
    } else {
      // Cross-class: convert on the source side when dtypes differ, then move.
      ArrayPtr staged = src;
      if (head_.second != key.second) {
        const Key skey(head_.first, key.second);
        staged = materialize(skey, src->context());
        if (!current_.count(skey)) {
          src->wait_event(src->context(), async_flags);
          staged->copy_from(src.get());
        }
        current_.insert(skey);
      }
      ArraySynchronizer::synchronize(head_.first, staged.get(), key.first, dst.get(), async_flags);
    }
    current_.insert(key);
    return dst;
  }

public:
  explicit SyncedArray(Size_t size) : size_(size) {}
  Size_t size() const { return size_; }
  ArrayPtr cast_sp(dtypes dtype, const Context &ctx, bool write_only = false,
                   const int async_flags = AsyncFlag::NONE) {
    ArrayPtr a = sync(dtype, ctx, write_only, async_flags);
    head_ = Key(ctx.array_class, static_cast<int>(dtype));
    has_head_ = true;
    zeroing_ = filling_ = false;
    // every other materialisation is stale now
    for (auto it = arrays_.begin(); it != arrays_.end();)
      it = (it->first == head_) ? std::next(it) : arrays_.erase(it);
    current_.clear();
    return a;
  }
  Array *cast(dtypes dtype, const Context &ctx, bool write_only = false,
              const int async_flags = AsyncFlag::NONE) {
    return cast_sp(dtype, ctx, write_only, async_flags).get();
  }
  const Array *get(dtypes dtype, const Context &ctx, const int async_flags = AsyncFlag::NONE) {
    ArrayPtr a = sync(dtype, ctx, false, async_flags);
    if (!has_head_ || zeroing_ || filling_) {
      head_ = Key(ctx.array_class, static_cast<int>(dtype));
      has_head_ = true;
      zeroing_ = filling_ = false;
    }
    return a.get();
  }
  void zero() {
    arrays_.clear();
    current_.clear();
    has_head_ = true;
    zeroing_ = true;
    filling_ = false;
    head_ = Key("", 0);
  }
  void fill(float v) {
    arrays_.clear();
    current_.clear();
    has_head_ = true;
    zeroing_ = false;
    filling_ = true;
    fill_value_ = v;
    head_ = Key("", 0);
  }
  void clear() {
    arrays_.clear();
    current_.clear();
    has_head_ = false;
    zeroing_ = filling_ = false;
  }
  bool zeroing() const { return zeroing_; }
  // dtype of the up-to-date materialisation (the core's SyncedArray::dtype()
  // likewise raises for an array that holds nothing yet).
  dtypes dtype() const {
    NBLA_CHECK(has_head_ && !zeroing_ && !filling_ && !head_.first.empty(), error_code::unclassified,
               "Array is not initialized.");
    return static_cast<dtypes>(head_.second);
  }
};
typedef shared_ptr<SyncedArray> SyncedArrayPtr;

class NBLA_API NdArray {
  Shape_t shape_;
  Size_t size_;
  SyncedArrayPtr array_;

public:
  explicit NdArray(const Shape_t &shape = {})
      : shape_(shape), size_(compute_size_by_shape(shape)), array_(make_shared<SyncedArray>(size_)) {}
  const Shape_t &shape() const { return shape_; }
  Size_t size(Size_t axis = 0) const { return compute_size_by_shape(shape_, axis); }
  Size_t ndim() const { return static_cast<Size_t>(shape_.size()); }
  void reshape(const Shape_t &shape, bool force = false) {
    const Size_t n = compute_size_by_shape(shape);
    if (n != size_) {
      NBLA_CHECK(force, error_code::value, "reshape changes the total size");
      size_ = n;
      array_ = make_shared<SyncedArray>(n);
    }
    shape_ = shape;
  }
  SyncedArrayPtr array() { return array_; }
  void zero() { array_->zero(); }
  void fill(float v) { array_->fill(v); }
  Array *cast(dtypes dtype, const Context &ctx, bool write_only = false,
              const int async_flags = AsyncFlag::NONE) {
    return array_->cast(dtype, ctx, write_only, async_flags);
  }
  const Array *get(dtypes dtype, const Context &ctx, const int async_flags = AsyncFlag::NONE) {
    return array_->get(dtype, ctx, async_flags);
  }
};
typedef shared_ptr<NdArray> NdArrayPtr;

// (Variable API used by the Function bodies:
// src/nbla/cuda/function/generic/layer_normalization.cu:91-93 and
// group_normalization.cu:57-62.)
class NBLA_API Variable {
  Shape_t shape_;
  NdArrayPtr data_, grad_;

public:
  explicit Variable(const Shape_t &shape = {})
      : shape_(shape), data_(make_shared<NdArray>(shape)), grad_(make_shared<NdArray>(shape)) {}
  const Shape_t &shape() const { return shape_; }
  Shape_t strides() const {
    Shape_t s(shape_.size(), 1);
    for (int i = static_cast<int>(shape_.size()) - 2; i >= 0; --i) s[i] = s[i + 1] * shape_[i + 1];
    return s;
  }
  Size_t ndim() const { return static_cast<Size_t>(shape_.size()); }
  Size_t size(Size_t axis = 0) const { return compute_size_by_shape(shape_, axis); }
  void reshape(const Shape_t &shape, bool force) {
    shape_ = shape;
    data_->reshape(shape, force);
    grad_->reshape(shape, force);
  }
  NdArrayPtr data() { return data_; }
  NdArrayPtr grad() { return grad_; }
  template <typename T> const T *get_data_pointer(const Context &ctx) {
    return data_->get(get_dtype<T>(), ctx)->template const_pointer<T>();
  }
  template <typename T> const T *get_grad_pointer(const Context &ctx) {
    return grad_->get(get_dtype<T>(), ctx)->template const_pointer<T>();
  }
  template <typename T> T *cast_data_and_get_pointer(const Context &ctx, bool write_only = false) {
    return data_->cast(get_dtype<T>(), ctx, write_only)->template pointer<T>();
  }
  template <typename T> T *cast_grad_and_get_pointer(const Context &ctx, bool write_only = false) {
    return grad_->cast(get_dtype<T>(), ctx, write_only)->template pointer<T>();
  }
};
typedef shared_ptr<Variable> VariablePtr;
typedef vector<Variable *> Variables; // function_impl.cu.tmpl:63-64

// ---------------------------------------------------------------- Function
// (virtuals at include/nbla/cuda/function/batch_normalization.hpp:63-84.)
class NBLA_API Function {
protected:
  Context ctx_;
  shared_ptr<Function> fall_back_func_;
  bool called_setup_ = false;

public:
  explicit Function(const Context &ctx) : ctx_(ctx) {}
  virtual ~Function() {}
  virtual string name() = 0;
  virtual vector<string> allowed_array_classes() = 0;
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  Context context() const { return ctx_; }

  void setup(const Variables &inputs, const Variables &outputs) {
    if (fall_back_func_) fall_back_func_.reset();
    const vector<string> allowed = allowed_array_classes();
    NBLA_CHECK(std::find(allowed.begin(), allowed.end(), ctx_.array_class) != allowed.end(),
               error_code::value, "Array class '%s' is not allowed in %s.",
               ctx_.array_class.c_str(), name().c_str());
    NBLA_CHECK(static_cast<int>(inputs.size()) >= min_inputs(), error_code::value,
               "%s needs at least %d inputs (given %zu).", name().c_str(), min_inputs(),
               inputs.size());
    NBLA_CHECK(static_cast<int>(outputs.size()) >= min_outputs(), error_code::value,
               "%s needs at least %d outputs (given %zu).", name().c_str(), min_outputs(),
               outputs.size());
    setup_impl(inputs, outputs);
    called_setup_ = true;
  }
  void forward(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(called_setup_, error_code::runtime, "%s: setup() was not called.", name().c_str());
    if (fall_back_func_) return fall_back_func_->forward(inputs, outputs);
    forward_impl(inputs, outputs);
  }
  void backward(const Variables &inputs, const Variables &outputs,
                const vector<bool> &propagate_down, const vector<bool> &accum) {
    NBLA_CHECK(called_setup_, error_code::runtime, "%s: setup() was not called.", name().c_str());
    NBLA_CHECK(propagate_down.size() == inputs.size() && accum.size() == inputs.size(),
               error_code::value, "propagate_down/accum must have one flag per input.");
    if (fall_back_func_) return fall_back_func_->backward(inputs, outputs, propagate_down, accum);
    backward_impl(inputs, outputs, propagate_down, accum);
  }
  void recompute(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(called_setup_, error_code::runtime, "%s: setup() was not called.", name().c_str());
    if (fall_back_func_) return fall_back_func_->recompute(inputs, outputs);
    recompute_impl(inputs, outputs);
  }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) = 0;
  virtual void forward_impl(const Variables &inputs, const Variables &outputs) = 0;
  virtual void backward_impl(const Variables &inputs, const Variables &outputs,
                             const vector<bool> &propagate_down, const vector<bool> &accum) = 0;
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs) {
    forward_impl(inputs, outputs);
  }
};
typedef shared_ptr<Function> FunctionPtr;

// ---------------------------------------------------------------- registry
// (NBLA_REGISTER_FUNCTION_IMPL(Base, Impl, "backend:type_config", argtypes...)
// at src/nbla/cuda/init.cpp.tmpl:223-234; creation walks Context.backend in
// order, python/src/nnabla_ext/cudnn/__init__.py:52-63.)
template <typename... Args> class FunctionRegistry {
public:
  typedef std::function<FunctionPtr(const Context &, Args...)> Creator;
  std::map<string, Creator> creators;
  std::mutex mu;
  void add(const string &backend, Creator c) {
    std::lock_guard<std::mutex> lock(mu);
    creators[backend] = c;
  }
  FunctionPtr create(const string &fname, const Context &ctx, Args... args) {
    Creator c;
    {
      std::lock_guard<std::mutex> lock(mu);
      for (const string &b : ctx.backend) {
        auto it = creators.find(b);
        if (it != creators.end()) {
          c = it->second;
          break;
        }
      }
    }
    NBLA_CHECK(c, error_code::unclassified,
               "No implementation of %s is registered for %s (this build registers the "
               "normalization functions under 'hip:float' and 'hip:half' only).",
               fname.c_str(), ctx.to_string().c_str());
    return c(ctx, args...);
  }
};

#define NBLA_REGISTER_FUNCTION_HEADER(NAME, ...)                                       \
  NBLA_API ::nbla::FunctionRegistry<__VA_ARGS__> &get_##NAME##Registry();              \
  template <typename... A> ::nbla::FunctionPtr create_##NAME(const ::nbla::Context &ctx, A... a) { \
    return get_##NAME##Registry().create(#NAME, ctx, a...);                            \
  }

#define NBLA_REGISTER_FUNCTION_SOURCE(NAME, ...)                                       \
  ::nbla::FunctionRegistry<__VA_ARGS__> &get_##NAME##Registry() {                      \
    static ::nbla::FunctionRegistry<__VA_ARGS__> registry;                             \
    return registry;                                                                   \
  }

#define NBLA_REGISTER_FUNCTION_IMPL(BASE, CLS, BACKEND, ...)                           \
  get_##BASE##Registry().add(BACKEND, [](const ::nbla::Context &ctx, auto... a) {      \
    return ::nbla::FunctionPtr(new CLS(ctx, a...));                                    \
  })

// ---------------------------------------------------------------- backends
// (BackendBase as subclassed by `Cuda`, include/nbla/cuda/cuda.hpp:49-187;
// NBLA_REGISTER_BACKEND at src/nbla/cuda/init.cpp.tmpl:89.)
class NBLA_API BackendBase {
public:
  virtual ~BackendBase() {}
  virtual vector<string> array_classes() const = 0;
  virtual void device_synchronize(const string &device) = 0;
  virtual void default_stream_synchronize(const string &device) = 0;
};

class NBLA_API BackendUtils {
public:
  typedef std::function<BackendBase *()> Getter;
  static std::map<string, Getter> &registry() {
    static std::map<string, Getter> r;
    return r;
  }
  static void add_backend(const string &name, Getter g) { registry()[name] = g; }
  static BackendBase *get(const string &name) {
    auto it = registry().find(name);
    NBLA_CHECK(it != registry().end(), error_code::unclassified, "backend '%s' is not registered",
               name.c_str());
    return it->second();
  }
  static vector<string> array_classes(const Context &ctx) {
    const string b = ctx.backend.empty() ? "cpu" : ctx.backend[0].substr(0, ctx.backend[0].find(':'));
    return get(b)->array_classes();
  }
};
#define NBLA_REGISTER_BACKEND(NAME, GETTER) ::nbla::BackendUtils::add_backend(NAME, GETTER)

class NBLA_API Cpu : public BackendBase {
public:
  vector<string> array_classes() const override { return {"CpuArray"}; }
  void device_synchronize(const string &) override {}
  void default_stream_synchronize(const string &) override {}
};

// Registers the "cpu" backend and the CpuArray class (idempotent).
inline void init_cpu() {
  static std::once_flag once;
  std::call_once(once, [] {
    NBLA_REGISTER_BACKEND("cpu", [] { return static_cast<BackendBase *>(SingletonManager::get<Cpu>()); });
    ArrayCreator::add_creator("CpuArray", [](Size_t s, dtypes d, const Context &c) -> Array * {
      return new CpuArray(s, d, c);
    });
    ArraySynchronizer::add_synchronizer("CpuArray", "CpuArray", [](Array *src, Array *dst, const int) {
      dst->copy_from(src);
    });
  });
}

} // namespace nbla
