// TensorNormalizationHip<T>: "hip" implementation of TensorNormalization with
// the interface of TensorNormalizationCuda<T>
// (include/nbla/cuda/function/tensor_normalization.hpp:22-46).  The reference
// class forwards to the core's composite (transposes around
// BatchNormalization); here the kept axes, when adjacent, map straight onto the
// BatchNormalization kernels' [size0, C, size2] view and nothing is transposed.
#pragma once

#include <nbla/function/tensor_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/utils/axis_adaptor.hpp>

namespace nbla {

template <typename T> class TensorNormalizationHip : public TensorNormalization<T> {
protected:
  int device_;
  Size_t size0_ = 1, size1_ = 1, size2_ = 1;
  Variable mean_, var_; // float32 statistics kept for backward
  Variable workspace_;
  size_t workspace_bytes_ = 0;
  // Kept axes that are not adjacent: permuted copies of x / dy / y / dx, alive
  // only inside a call.
  AxisAdaptor adaptor_;
  Variable adapt_a_, adapt_b_, adapt_c_;

public:
  TensorNormalizationHip(const Context &ctx, const vector<int> &axes, float eps, bool no_scale,
                         bool no_bias)
      : TensorNormalization<T>(ctx, axes, eps, no_scale, no_bias),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~TensorNormalizationHip() {}
  virtual string name() { return "TensorNormalizationHip"; }
  virtual vector<string> allowed_array_classes() {
    return SingletonManager::get<Hip>()->array_classes();
  }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs,
                             const vector<bool> &propagate_down, const vector<bool> &accum);
};
} // namespace nbla
