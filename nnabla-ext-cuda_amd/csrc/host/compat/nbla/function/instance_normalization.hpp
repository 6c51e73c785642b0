// Stand-in for the core's nbla/function/instance_normalization.hpp (arguments
// and shapes only; see core_min.hpp).  Members as read by
// src/nbla/cuda/function/generic/instance_normalization.cu:31-97,160-170.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(InstanceNormalization, int, const vector<int> &, float, bool, bool);

template <typename T> class InstanceNormalization : public Function {
protected:
  int channel_axis_;
  vector<int> batch_axis_;
  float eps_;
  bool no_scale_;
  bool no_bias_;
  int beta_idx_, gamma_idx_;
  // A parameter whose batch extent is 1 while x's is larger is shared by the
  // whole batch (index row % channels); otherwise it is per sample.
  bool need_beta_broadcast_, need_gamma_broadcast_;

public:
  InstanceNormalization(const Context &ctx, int channel_axis, const vector<int> &batch_axis,
                        float eps, bool no_scale, bool no_bias)
      : Function(ctx), channel_axis_(channel_axis), batch_axis_(batch_axis), eps_(eps),
        no_scale_(no_scale), no_bias_(no_bias), beta_idx_(-1), gamma_idx_(-1),
        need_beta_broadcast_(true), need_gamma_broadcast_(true) {}
  virtual ~InstanceNormalization() {}
  string name() override { return "InstanceNormalization"; }

protected:
  void setup_shapes(const Variables &inputs, const Variables &outputs) {
    const size_t n_in = 1 + (no_bias_ ? 0 : 1) + (no_scale_ ? 0 : 1);
    NBLA_CHECK(inputs.size() == n_in, error_code::value,
               "InstanceNormalization expects %zu inputs, given %zu.", n_in, inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "InstanceNormalization has 1 or 3 outputs.");
    const Shape_t shape = inputs[0]->shape();
    const int ndim = static_cast<int>(shape.size());
    if (channel_axis_ < 0) channel_axis_ += ndim;
    NBLA_CHECK(channel_axis_ >= 0 && channel_axis_ < ndim, error_code::value,
               "channel_axis out of range.");
    Size_t batch = 1;
    for (int &b : batch_axis_) {
      if (b < 0) b += ndim;
      NBLA_CHECK(b >= 0 && b < ndim && b != channel_axis_, error_code::value,
                 "batch_axis out of range or equal to channel_axis.");
      batch *= shape[b];
    }
    const Size_t c = shape[channel_axis_];
    beta_idx_ = no_bias_ ? -1 : 1;
    gamma_idx_ = no_scale_ ? -1 : (no_bias_ ? 1 : 2);
    auto check_param = [&](int idx, bool &bc) {
      if (idx < 0) return;
      const Size_t n = inputs[idx]->size();
      NBLA_CHECK(n == c || n == batch * c, error_code::value,
                 "beta/gamma must have channels (%lld) or batch*channels (%lld) elements.",
                 static_cast<long long>(c), static_cast<long long>(batch * c));
      bc = (n == c);
    };
    check_param(beta_idx_, need_beta_broadcast_);
    check_param(gamma_idx_, need_gamma_broadcast_);
    outputs[0]->reshape(shape, true);
    if (outputs.size() == 3) {
      Shape_t stat_shape = shape;
      for (int i = 0; i < ndim; ++i) {
        const bool is_batch = std::find(batch_axis_.begin(), batch_axis_.end(), i) != batch_axis_.end();
        if (!is_batch && i != channel_axis_) stat_shape[i] = 1;
      }
      outputs[1]->reshape(stat_shape, true);
      outputs[2]->reshape(stat_shape, true);
    }
  }
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    setup_shapes(inputs, outputs);
  }
};
} // namespace nbla
