// Stand-in for the core's nbla/function/group_normalization.hpp (arguments and
// shapes only; see core_min.hpp).  Members as read by
// src/nbla/cuda/function/generic/group_normalization.cu:30-90.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(GroupNormalization, int, int, const vector<int> &, float, bool, bool);

template <typename T> class GroupNormalization : public Function {
protected:
  int num_groups_;
  int channel_axis_;
  vector<int> batch_axis_;
  float eps_;
  bool no_scale_;
  bool no_bias_;

public:
  GroupNormalization(const Context &ctx, int num_groups, int channel_axis,
                     const vector<int> &batch_axis, float eps, bool no_scale, bool no_bias)
      : Function(ctx), num_groups_(num_groups), channel_axis_(channel_axis),
        batch_axis_(batch_axis), eps_(eps), no_scale_(no_scale), no_bias_(no_bias) {}
  virtual ~GroupNormalization() {}
  string name() override { return "GroupNormalization"; }

protected:
  // y like x; with three outputs, mean and var have x's rank with the channel
  // axis holding num_groups and every axis that is neither batch nor channel 1.
  void setup_shapes(const Variables &inputs, const Variables &outputs) {
    const size_t n_in = 1 + (no_bias_ ? 0 : 1) + (no_scale_ ? 0 : 1);
    NBLA_CHECK(inputs.size() == n_in, error_code::value,
               "GroupNormalization expects %zu inputs, given %zu.", n_in, inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "GroupNormalization has 1 or 3 outputs.");
    const Shape_t shape = inputs[0]->shape();
    const int ndim = static_cast<int>(shape.size());
    if (channel_axis_ < 0) channel_axis_ += ndim;
    NBLA_CHECK(channel_axis_ >= 0 && channel_axis_ < ndim, error_code::value,
               "channel_axis out of range.");
    for (int &b : batch_axis_) {
      if (b < 0) b += ndim;
      NBLA_CHECK(b >= 0 && b < ndim && b != channel_axis_, error_code::value,
                 "batch_axis out of range or equal to channel_axis.");
    }
    const Size_t c = shape[channel_axis_];
    NBLA_CHECK(num_groups_ > 0 && c % num_groups_ == 0, error_code::value,
               "The channel dimension (%lld) must be divisible by num_groups (%d).",
               static_cast<long long>(c), num_groups_);
    for (size_t i = 1; i < inputs.size(); ++i)
      NBLA_CHECK(inputs[i]->size() == c, error_code::value,
                 "beta/gamma must have one element per channel.");
    outputs[0]->reshape(shape, true);
    if (outputs.size() == 3) {
      Shape_t stat_shape = shape;
      for (int i = 0; i < ndim; ++i) {
        const bool is_batch = std::find(batch_axis_.begin(), batch_axis_.end(), i) != batch_axis_.end();
        if (!is_batch) stat_shape[i] = 1;
      }
      stat_shape[channel_axis_] = num_groups_;
      outputs[1]->reshape(stat_shape, true);
      outputs[2]->reshape(stat_shape, true);
    }
  }
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    setup_shapes(inputs, outputs);
  }
};
} // namespace nbla
