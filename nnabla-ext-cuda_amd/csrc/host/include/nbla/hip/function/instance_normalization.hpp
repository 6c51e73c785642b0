// InstanceNormalizationHip<T>: "hip" implementation of InstanceNormalization
// with the interface of InstanceNormalizationCuda<T>
// (include/nbla/cuda/function/instance_normalization.hpp:25-74).
#pragma once

#include <nbla/function/instance_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/utils/param_stage.hpp>
#include <nbla/hip/utils/channel_layout.hpp>

namespace nbla {

template <typename T> class InstanceNormalizationHip : public InstanceNormalization<T> {
protected:
  int device_;
  Size_t batch_size_ = 0, channel_size_ = 0, spatial_size_ = 0;
  bool channel_last_ = false; // x is [batch..., spatial..., channel]
  Variable mean_, var_;   // float32 per-(n, c) statistics kept for backward
  Variable workspace_;
  Variable stage_; // float32 staging of parameters / statistics stored in half (ParamStage)
  size_t workspace_bytes_ = 0;
  // Layouts that are neither channel-first nor channel-last: permuted copies
  // of x / dy / y / dx, of the statistics and of per-sample parameters, alive
  // only inside a call.
  ChannelLayout layout_;
  Variable adapt_a_, adapt_b_, adapt_c_;
  Variable stat_a_, stat_b_, stat_c_, stat_d_, stat_e_, stat_f_, stat_g_;

public:
  InstanceNormalizationHip(const Context &ctx, int channel_axis, const vector<int> &batch_axis,
                           float eps, bool no_scale, bool no_bias)
      : InstanceNormalization<T>(ctx, channel_axis, batch_axis, eps, no_scale, no_bias),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~InstanceNormalizationHip() {}
  virtual string name() { return "InstanceNormalizationHip"; }
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
