// Stand-in for the core's nbla/function/batch_normalization.hpp: the base class
// the backend implementations derive from.  It owns the argument checks and
// the shape bookkeeping the reference reads from `this->` (size0_, size1_,
// size2_, size02_, size12_, b_idx_, g_idx_, m_idx_, v_idx_, mean_, var_:
// src/nbla/cuda/function/generic/batch_normalization.cu:34-35,53-55,120-143)
// and carries no arithmetic.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(BatchNormalization, const vector<int> &, float, float, bool, bool, bool);

template <typename T> class BatchNormalization : public Function {
protected:
  vector<int> axes_;
  float decay_rate_;
  float eps_;
  bool batch_stat_;
  bool no_scale_;
  bool no_bias_;
  int b_idx_, g_idx_, m_idx_, v_idx_;
  Variable mean_, var_;
  Size_t size0_, size1_, size2_, size02_, size12_;

public:
  BatchNormalization(const Context &ctx, const vector<int> axes, float decay_rate, float eps,
                     bool batch_stat, bool no_scale, bool no_bias)
      : Function(ctx), axes_(axes), decay_rate_(decay_rate), eps_(eps), batch_stat_(batch_stat),
        no_scale_(no_scale), no_bias_(no_bias) {}
  virtual ~BatchNormalization() {}
  string name() override { return "BatchNormalization"; }
  int min_inputs() override { return 3; }
  int min_outputs() override { return 1; }

protected:
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    NBLA_CHECK(axes_.size() == 1, error_code::not_implemented,
               "Specifying more than one axis is not supported.");
    const size_t n_in = 3 + (no_bias_ ? 0 : 1) + (no_scale_ ? 0 : 1);
    NBLA_CHECK(inputs.size() == n_in, error_code::value,
               "BatchNormalization expects %zu inputs (x%s%s, mean, var), given %zu.", n_in,
               no_bias_ ? "" : ", beta", no_scale_ ? "" : ", gamma", inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "BatchNormalization has 1 or 3 outputs.");
    NBLA_CHECK(batch_stat_ || outputs.size() == 1, error_code::value,
               "Mean/variance outputs require batch_stat=true.");
    b_idx_ = no_bias_ ? -1 : 1;
    g_idx_ = no_scale_ ? -1 : (no_bias_ ? 1 : 2);
    m_idx_ = static_cast<int>(n_in) - 2;
    v_idx_ = m_idx_ + 1;

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
    size02_ = size0_ * size2_;
    size12_ = size1_ * size2_;
    for (size_t i = 1; i < inputs.size(); ++i) {
      NBLA_CHECK(inputs[i]->size() == size1_, error_code::value,
                 "Parameter %zu must have %lld elements (given %lld).", i,
                 static_cast<long long>(size1_), static_cast<long long>(inputs[i]->size()));
    }
    NBLA_CHECK(!batch_stat_ || size02_ >= 1, error_code::value, "empty reduction");
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
