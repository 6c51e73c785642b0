// ParamStage: parameter and statistics arrays of a "hip:half" function that
// the graph stores in half precision.
//
// The kernel layer takes gamma, beta, statistics and their gradients as
// float32 (the reference's cudnn context does the same for half activations,
// cudnn/function/generic/batch_normalization.cu:94-99).  The reference's plain
// cuda:half type config keeps them in Tc = half
// (layer_normalization.cu:91-93, batch_normalization.cu:124-143): fetching such
// an array as float through the core would convert it with a kernel of its
// own, hold a second copy, and leave an array the function writes - running
// statistics, gradients, exposed mean / var - stored as float from then on.
// Here an array whose up-to-date copy is half is read and written where it
// lies: everything the call reads goes to a float32 staging buffer in one
// launch before the kernels (nblahip_stage_params), everything it wrote goes
// back in one launch after them, and the stored arrays keep their type.
// Arrays stored as float (and every array of a "hip:float" function) pass
// through untouched.  An output that holds nothing yet is written in half when
// the function's parameters are half (follow(): the first half input decides).
#pragma once

#include <nbla/hip/common.hpp>
#include <nbla/nd_array.hpp>
#include <nbla/variable.hpp>

#include <vector>

namespace nbla {

class ParamStage {
  Context ctx_;
  bool enabled_ = false; // hip:half functions only
  bool half_outputs_ = false;
  float *base_ = nullptr;
  Size_t used_ = 0, capacity_ = 0;
  struct Seg {
    void *half_ptr;
    float *staged;
    Size_t n;
  };
  std::vector<Seg> loads_, stores_;

  static bool stored_as_half(NdArray *a) {
    try {
      return a->array()->dtype() == dtypes::HALF;
    } catch (...) { // nothing stored yet
      return false;
    }
  }
  static bool holds_nothing(NdArray *a) {
    try {
      (void)a->array()->dtype();
      return false;
    } catch (...) {
      return true;
    }
  }
  float *take(Size_t n) {
    const Size_t padded = (n + 63) / 64 * 64;
    NBLA_CHECK(used_ + padded <= capacity_, error_code::memory,
               "ParamStage: staging buffer of %lld floats exhausted.",
               static_cast<long long>(capacity_));
    float *p = base_ + used_;
    used_ += padded;
    return p;
  }
  void run(const std::vector<Seg> &segs, bool to_float) {
    for (size_t first = 0; first < segs.size(); first += 16) {
      const void *src[16];
      void *dst[16];
      int64_t n[16];
      int count = 0;
      for (size_t i = first; i < segs.size() && count < 16; ++i, ++count) {
        src[count] = to_float ? segs[i].half_ptr : static_cast<const void *>(segs[i].staged);
        dst[count] = to_float ? static_cast<void *>(segs[i].staged) : segs[i].half_ptr;
        n[count] = segs[i].n;
      }
      NBLA_HIP_CHECK(nblahip_stage_params(count, src, to_float ? NBLAHIP_F16 : NBLAHIP_F32, dst,
                                          to_float ? NBLAHIP_F32 : NBLAHIP_F16, n, nullptr));
    }
  }

public:
  // Floats of staging a call with these array sizes may need (each padded).
  static Size_t capacity_for(const std::vector<Size_t> &sizes) {
    Size_t total = 0;
    for (Size_t n : sizes) total += (n + 63) / 64 * 64;
    return total;
  }

  // half_type: the function's T is Half.  buffer: a float Variable of at least
  // capacity_for(...) elements owned by the function.
  void begin(const Context &ctx, bool half_type, Variable *buffer) {
    ctx_ = ctx;
    enabled_ = half_type;
    half_outputs_ = false;
    used_ = 0;
    loads_.clear();
    stores_.clear();
    capacity_ = buffer ? buffer->size() : 0;
    base_ = nullptr;
    if (enabled_ && capacity_ > 0) base_ = buffer->cast_data_and_get_pointer<float>(ctx_, true);
  }

  // An array the kernels read.
  const float *in(NdArray *a) {
    if (!a) return nullptr;
    if (!enabled_ || !stored_as_half(a)) return a->get(dtypes::FLOAT, ctx_)->const_pointer<float>();
    half_outputs_ = true;
    Seg s{const_cast<void *>(a->get(dtypes::HALF, ctx_)->const_pointer<void>()), take(a->size()),
          a->size()};
    loads_.push_back(s);
    return s.staged;
  }
  const float *in(Variable *v, bool grad = false) {
    return v ? in(grad ? v->grad().get() : v->data().get()) : nullptr;
  }

  // An array the kernels write; keep: they read it first (accumulation, running
  // statistics).
  float *out(NdArray *a, bool keep) {
    if (!a) return nullptr;
    const bool half = enabled_ && (stored_as_half(a) || (half_outputs_ && holds_nothing(a)) ||
                                   (half_outputs_ && !keep));
    if (!half) return a->cast(dtypes::FLOAT, ctx_, !keep)->pointer<float>();
    Seg s{a->cast(dtypes::HALF, ctx_, !keep)->pointer<void>(), take(a->size()), a->size()};
    if (keep) loads_.push_back(s);
    stores_.push_back(s);
    return s.staged;
  }
  float *out(Variable *v, bool keep, bool grad = false) {
    return v ? out(grad ? v->grad().get() : v->data().get(), keep) : nullptr;
  }

  void load() {
    if (!loads_.empty()) run(loads_, true);
  }
  void store() {
    if (!stores_.empty()) run(stores_, false);
  }
  bool staging() const { return !loads_.empty() || !stores_.empty(); }
};

} // namespace nbla
