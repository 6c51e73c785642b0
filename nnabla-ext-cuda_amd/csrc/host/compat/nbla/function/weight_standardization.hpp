// Stand-in for the core's nbla/function/weight_standardization.hpp (arguments
// and shapes only; see core_min.hpp).  Constructor arguments as
// include/nbla/cuda/function/weight_standardization.hpp:26-28 passes them on.
// y = (w - mean) / sqrt(var + eps) with mean and variance over every axis but
// channel_axis; the optional outputs mean and var keep that axis.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(WeightStandardization, int, float);

template <typename T> class WeightStandardization : public Function {
protected:
  int channel_axis_;
  float eps_;

public:
  WeightStandardization(const Context &ctx, int channel_axis, float eps)
      : Function(ctx), channel_axis_(channel_axis), eps_(eps) {}
  virtual ~WeightStandardization() {}
  string name() override { return "WeightStandardization"; }

protected:
  void setup_shapes(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(inputs.size() == 1, error_code::value,
               "WeightStandardization expects 1 input, given %zu.", inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "WeightStandardization has 1 or 3 outputs.");
    const Shape_t shape = inputs[0]->shape();
    const int ndim = static_cast<int>(shape.size());
    if (channel_axis_ < 0) channel_axis_ += ndim;
    NBLA_CHECK(channel_axis_ >= 0 && channel_axis_ < ndim, error_code::value,
               "channel_axis out of range.");
    outputs[0]->reshape(shape, true);
    if (outputs.size() == 3) {
      Shape_t stat_shape(ndim, 1);
      stat_shape[channel_axis_] = shape[channel_axis_];
      outputs[1]->reshape(stat_shape, true);
      outputs[2]->reshape(stat_shape, true);
    }
  }
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    setup_shapes(inputs, outputs);
  }
};
} // namespace nbla
