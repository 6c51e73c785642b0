// GroupNormalizationHip<T>: "hip" implementation of GroupNormalization with the
// interface of GroupNormalizationCuda<T>
// (include/nbla/cuda/function/group_normalization.hpp:26-72).
#pragma once

#include <nbla/function/group_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/utils/param_stage.hpp>
#include <nbla/hip/utils/channel_layout.hpp>

namespace nbla {

template <typename T> class GroupNormalizationHip : public GroupNormalization<T> {
protected:
  int device_;
  Size_t batch_size_ = 0, channel_size_ = 0, spatial_size_ = 0;
  bool channel_last_ = false; // x is [batch..., spatial..., channel]
  Variable mean_, var_;   // float32 per-(n, group) statistics kept for backward
  Variable workspace_;
  Variable stage_; // float32 staging of parameters / statistics stored in half (ParamStage)
  size_t workspace_bytes_ = 0;
  // Layouts that are neither channel-first nor channel-last: permuted copies
  // of x / dy / y / dx and of the statistics, alive only inside a call.
  ChannelLayout layout_;
  Variable adapt_a_, adapt_b_, adapt_c_, stat_a_, stat_b_, stat_c_, stat_d_;

public:
  GroupNormalizationHip(const Context &ctx, int num_groups, int channel_axis,
                        const vector<int> &batch_axis, float eps, bool no_scale, bool no_bias)
      : GroupNormalization<T>(ctx, num_groups, channel_axis, batch_axis, eps, no_scale, no_bias),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~GroupNormalizationHip() {}
  virtual string name() { return "GroupNormalizationHip"; }
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
