// Stand-in for the core's nbla/function/tensor_normalization.hpp (arguments
// and shapes only; see core_min.hpp).  Constructor arguments as
// include/nbla/cuda/function/tensor_normalization.hpp:26-28 passes them on.
// `axes` are the axes the statistics KEEP (as BatchNormalization's axes): for
// x[B, C, H, W] and axes = {0, 1} mean and variance have shape [B, C, 1, 1],
// and so have beta and gamma.
#pragma once
#include <nbla/core_min.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(TensorNormalization, const vector<int> &, float, bool, bool);

template <typename T> class TensorNormalization : public Function {
protected:
  vector<int> axes_;
  float eps_;
  bool no_scale_;
  bool no_bias_;
  int beta_idx_, gamma_idx_;
  Shape_t stat_shape_;

public:
  TensorNormalization(const Context &ctx, const vector<int> &axes, float eps, bool no_scale,
                      bool no_bias)
      : Function(ctx), axes_(axes), eps_(eps), no_scale_(no_scale), no_bias_(no_bias),
        beta_idx_(-1), gamma_idx_(-1) {}
  virtual ~TensorNormalization() {}
  string name() override { return "TensorNormalization"; }

protected:
  void setup_shapes(const Variables &inputs, const Variables &outputs) {
    const size_t n_in = 1 + (no_bias_ ? 0 : 1) + (no_scale_ ? 0 : 1);
    NBLA_CHECK(inputs.size() == n_in, error_code::value,
               "TensorNormalization expects %zu inputs, given %zu.", n_in, inputs.size());
    NBLA_CHECK(outputs.size() == 1 || outputs.size() == 3, error_code::value,
               "TensorNormalization has 1 or 3 outputs.");
    const Shape_t shape = inputs[0]->shape();
    const int ndim = static_cast<int>(shape.size());
    NBLA_CHECK(!axes_.empty(), error_code::value, "TensorNormalization needs at least one axis.");
    for (int &a : axes_) {
      if (a < 0) a += ndim;
      NBLA_CHECK(a >= 0 && a < ndim, error_code::value, "axes out of range.");
    }
    std::sort(axes_.begin(), axes_.end());
    NBLA_CHECK(std::adjacent_find(axes_.begin(), axes_.end()) == axes_.end(), error_code::value,
               "axes must be distinct.");
    stat_shape_.assign(ndim, 1);
    Size_t stat_size = 1;
    for (int a : axes_) {
      stat_shape_[a] = shape[a];
      stat_size *= shape[a];
    }
    beta_idx_ = no_bias_ ? -1 : 1;
    gamma_idx_ = no_scale_ ? -1 : (no_bias_ ? 1 : 2);
    for (int idx : {beta_idx_, gamma_idx_}) {
      if (idx < 0) continue;
      NBLA_CHECK(inputs[idx]->size() == stat_size, error_code::value,
                 "beta/gamma must have %lld elements (the kept axes), given %lld.",
                 static_cast<long long>(stat_size), static_cast<long long>(inputs[idx]->size()));
    }
    outputs[0]->reshape(shape, true);
    if (outputs.size() == 3) {
      outputs[1]->reshape(stat_shape_, true);
      outputs[2]->reshape(stat_shape_, true);
    }
  }
  void setup_impl(const Variables &inputs, const Variables &outputs) override {
    setup_shapes(inputs, outputs);
  }
};
} // namespace nbla
