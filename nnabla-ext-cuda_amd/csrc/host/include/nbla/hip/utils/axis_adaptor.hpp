// AxisAdaptor: brings a tensor to the axis order the normalization kernels
// read (chosen "front" axes first, every other axis after them in its own
// order) with a device permutation, and back.  It plays the part of the core's
// ChannelFirstAdaptor, through which the reference runs every layout its
// kernels do not read in place (src/nbla/cuda/function/generic/
// group_normalization.cu:40-55,93-109,203-224, instance_normalization.cu:40-51,
// 81-94,187-207), and of the core's transposing composites behind
// LayerNormalization with non-leading batch axes (layer_normalization.cu:43-51)
// and TensorNormalization (tensor_normalization.cu:22-46).  Nothing here
// touches the host: both directions are one kernel launch (nblahip_permute).
#pragma once

#include <nbla/hip/common.hpp>
#include <nbla/variable.hpp>

#include <algorithm>
#include <vector>

namespace nbla {

class AxisAdaptor {
  std::vector<int64_t> shape_, kernel_shape_;
  std::vector<int> perm_, inverse_;
  bool needed_ = false;

public:
  // front: axes of `shape` that lead the kernel layout, in the order given.
  // back_first == false: kernel layout = front axes, then the rest ascending;
  // back_first == true : the rest ascending, then the front axes.
  void setup(const Shape_t &shape, const std::vector<int> &front, bool back_first = false) {
    const int nd = static_cast<int>(shape.size());
    NBLA_CHECK(nd <= 8, error_code::not_implemented,
               "The hip backend permutes tensors of at most 8 axes.");
    shape_.assign(shape.begin(), shape.end());
    std::vector<int> rest;
    for (int i = 0; i < nd; ++i)
      if (std::find(front.begin(), front.end(), i) == front.end()) rest.push_back(i);
    perm_.clear();
    if (back_first) perm_ = rest;
    perm_.insert(perm_.end(), front.begin(), front.end());
    if (!back_first) perm_.insert(perm_.end(), rest.begin(), rest.end());
    inverse_.assign(nd, 0);
    kernel_shape_.assign(nd, 1);
    // A permutation that only moves axes of extent 1 leaves memory as it is.
    std::vector<int> moved_a, moved_b;
    for (int i = 0; i < nd; ++i) {
      inverse_[perm_[i]] = i;
      kernel_shape_[i] = shape_[perm_[i]];
      if (shape_[i] != 1) moved_a.push_back(i);
      if (shape_[perm_[i]] != 1) moved_b.push_back(perm_[i]);
    }
    needed_ = moved_a != moved_b;
  }
  bool needed() const { return needed_; }

  // dst (kernel layout) = src (caller's layout)
  void to_kernel(const void *src, void *dst, int dtype) const {
    NBLA_HIP_CHECK(nblahip_permute(src, dst, static_cast<int>(shape_.size()), shape_.data(),
                                   perm_.data(), 0, dtype, nullptr));
  }
  // dst (caller's layout) = src (kernel layout), or += with accum
  void to_caller(const void *src, void *dst, bool accum, int dtype) const {
    NBLA_HIP_CHECK(nblahip_permute(src, dst, static_cast<int>(kernel_shape_.size()),
                                   kernel_shape_.data(), inverse_.data(), accum ? 1 : 0, dtype,
                                   nullptr));
  }
};

// n elements of write-only scratch of type T in a function-owned Variable.
template <typename T> inline T *adaptor_scratch(Variable &v, Size_t n, const Context &ctx) {
  v.reshape(Shape_t{n}, true);
  return v.cast_data_and_get_pointer<T>(ctx, true);
}
inline void adaptor_release(Variable &v) { v.data()->array()->clear(); }

} // namespace nbla
