// WeightStandardizationHip<T>: "hip" implementation of WeightStandardization
// with the interface of WeightStandardizationCuda<T>
// (include/nbla/cuda/function/weight_standardization.hpp:22-46), on the
// BatchNormalization kernels' [size0, C, size2] view without scale and bias.
#pragma once

#include <nbla/function/weight_standardization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class WeightStandardizationHip : public WeightStandardization<T> {
protected:
  int device_;
  Size_t size0_ = 1, size1_ = 1, size2_ = 1;
  Variable mean_, var_;
  Variable workspace_;
  size_t workspace_bytes_ = 0;

public:
  WeightStandardizationHip(const Context &ctx, int channel_axis, float eps)
      : WeightStandardization<T>(ctx, channel_axis, eps), device_(std::stoi(ctx.device_id)) {}
  virtual ~WeightStandardizationHip() {}
  virtual string name() { return "WeightStandardizationHip"; }
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
