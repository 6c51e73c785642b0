// Stand-in for the core's nbla/function/fused_batch_normalization.hpp: argument
// checks and shape bookkeeping only (see core_min.hpp).  Members as read by
// src/nbla/cuda/cudnn/function/generic/fused_batch_normalization.cu:40-52,
// 136-160 (axes_, decay_rate_, eps_, batch_stat_, nonlinearity_, mean_, var_).
// Inputs [x, beta, gamma, mean, var] or [x, beta, gamma, mean, var, z];
// outputs [y] or [y, batch_mean, batch_var].
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(FusedBatchNormalization, const vector<int> &, float, float, bool,
                              const string &);

template <typename T> class FusedBatchNormalization : public Function {
protected:
  vector<int> axes_;
  float decay_rate_;
  float eps_;
  bool batch_stat_;
  string nonlinearity_;
  Variable mean_, var_;
  Size_t size0_, size1_, size2_;

public:
  FusedBatchNormalization(const Context &ctx, const vector<int> axes, float decay_rate, float eps,
                          bool batch_stat, const string &nonlinearity)
      : Function(ctx), axes_(axes), decay_rate_(decay_rate), eps_(eps), batch_stat_(batch_stat),
        nonlinearity_(nonlinearity) {}
  virtual ~FusedBatchNormalization() {}
  string name() override { return "FusedBatchNormalization"; }
  int min_inputs() override { return 5; }
  int min_outputs() override { return 1; }

protected:
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    NBLA_CHECK(nonlinearity_ == "relu", error_code::not_implemented,
               "FusedBatchNormalization supports the nonlinearity \"relu\" only.");
    NBLA_CHECK(axes_.size() == 1, error_code::not_implemented,
               "Specifying more than one axis is not supported.");
    NBLA_CHECK(inputs.size() == 5 || inputs.size() == 6, error_code::value,
               "FusedBatchNormalization expects 5 or 6 inputs (x, beta, gamma, mean, var[, z]), "
               "given %zu.", inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "FusedBatchNormalization has 1 or 3 outputs.");
    NBLA_CHECK(batch_stat_ || outputs.size() == 1, error_code::value,
               "Mean/variance outputs require batch_stat=true.");
    const Shape_t shape = inputs[0]->shape();
    int axis = axes_[0];
    if (axis < 0) axis += static_cast<int>(shape.size());
    NBLA_CHECK(axis >= 0 && axis < static_cast<int>(shape.size()), error_code::value,
               "axes[0]=%d is out of range for a %zu-d input.", axes_[0], shape.size());
    axes_[0] = axis;
    size0_ = 1;
    for (int i = 0; i < axis; ++i) size0_ *= shape[i];
    size1_ = shape[axis];
    size2_ = inputs[0]->size(axis + 1);
    for (size_t i = 1; i < 5; ++i) {
      NBLA_CHECK(inputs[i]->size() == size1_, error_code::value,
                 "Parameter %zu must have %lld elements (given %lld).", i,
                 static_cast<long long>(size1_), static_cast<long long>(inputs[i]->size()));
    }
    if (inputs.size() == 6) {
      NBLA_CHECK(inputs[5]->shape() == shape, error_code::value,
                 "The residual input z must have the shape of x.");
    }
    NBLA_CHECK(!batch_stat_ || size0_ * size2_ >= 1, error_code::value, "empty reduction");
    outputs[0]->reshape(shape, true);
    Shape_t stat_shape(shape.size(), 1);
    stat_shape[axis] = size1_;
    if (outputs.size() == 3) {
      outputs[1]->reshape(stat_shape, true);
      outputs[2]->reshape(stat_shape, true);
    }
    mean_.reshape(stat_shape, true);
    var_.reshape(stat_shape, true);
  }
};
} // namespace nbla
