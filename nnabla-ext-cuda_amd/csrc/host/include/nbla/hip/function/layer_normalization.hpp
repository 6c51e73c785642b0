// LayerNormalizationHip<T>: "hip" implementation of LayerNormalization with the
// interface of LayerNormalizationCuda<T>
// (include/nbla/cuda/function/layer_normalization.hpp:25-55).
#pragma once

#include <nbla/function/layer_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/utils/axis_adaptor.hpp>
#include <nbla/hip/utils/param_stage.hpp>

namespace nbla {

template <typename T> class LayerNormalizationHip : public LayerNormalization<T> {
protected:
  int device_;
  Size_t batch_size_ = 0, reduce_size_ = 0;
  Variable mean_, var_;   // float32 row statistics kept for backward
  Variable workspace_;
  size_t workspace_bytes_ = 0;
  Variable stage_; // float32 staging of parameters / statistics stored in half (ParamStage)
  // Batch axes that are not the leading ones: permuted copies of x / dy / y /
  // dx, alive only inside a call.
  AxisAdaptor adaptor_;
  Variable adapt_a_, adapt_b_, adapt_c_;

public:
  LayerNormalizationHip(const Context &ctx, const vector<int> &batch_axis, float eps,
                        bool no_scale, bool no_bias)
      : LayerNormalization<T>(ctx, batch_axis, eps, no_scale, no_bias),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~LayerNormalizationHip() {}
  virtual string name() { return "LayerNormalizationHip"; }
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
