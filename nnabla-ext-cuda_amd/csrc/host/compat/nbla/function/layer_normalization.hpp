// Stand-in for the core's nbla/function/layer_normalization.hpp (arguments and
// shapes only; see core_min.hpp).  Members as read by
// src/nbla/cuda/function/generic/layer_normalization.cu:30-75.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(LayerNormalization, const vector<int> &, float, bool, bool);

template <typename T> class LayerNormalization : public Function {
protected:
  vector<int> batch_axis_;
  float eps_;
  bool no_scale_;
  bool no_bias_;

public:
  LayerNormalization(const Context &ctx, const vector<int> &batch_axis, float eps, bool no_scale,
                     bool no_bias)
      : Function(ctx), batch_axis_(batch_axis), eps_(eps), no_scale_(no_scale), no_bias_(no_bias) {}
  virtual ~LayerNormalization() {}
  string name() override { return "LayerNormalization"; }
  int min_inputs() override { return 1; }
  int min_outputs() override { return 1; }

protected:
  // Argument checks and output shapes: y like x; with three outputs, mean and
  // var keep the batch axes and collapse every other axis to 1.
  void setup_shapes(const Variables &inputs, const Variables &outputs) {
    const size_t n_in = 1 + (no_bias_ ? 0 : 1) + (no_scale_ ? 0 : 1);
    NBLA_CHECK(inputs.size() == n_in, error_code::value,
               "LayerNormalization expects %zu inputs, given %zu.", n_in, inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "LayerNormalization has 1 or 3 outputs.");
    const Shape_t shape = inputs[0]->shape();
    const int ndim = static_cast<int>(shape.size());
    NBLA_CHECK(!batch_axis_.empty(), error_code::value, "batch_axis must not be empty.");
    for (int &b : batch_axis_) {
      if (b < 0) b += ndim;
      NBLA_CHECK(b >= 0 && b < ndim, error_code::value, "batch_axis out of range.");
    }
    Shape_t stat_shape(shape.size(), 1), param_shape = shape;
    for (int b : batch_axis_) {
      stat_shape[b] = shape[b];
      param_shape[b] = 1;
    }
    const Size_t psize = compute_size_by_shape(param_shape);
    for (size_t i = 1; i < inputs.size(); ++i)
      NBLA_CHECK(inputs[i]->size() == psize, error_code::value,
                 "beta/gamma must have %lld elements.", static_cast<long long>(psize));
    outputs[0]->reshape(shape, true);
    if (outputs.size() == 3) {
      outputs[1]->reshape(stat_shape, true);
      outputs[2]->reshape(stat_shape, true);
    }
  }
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    setup_shapes(inputs, outputs);
  }
};
} // namespace nbla
