// FusedBatchNormalizationHip<T>: the "hip" implementation of
// FusedBatchNormalization (BatchNormalization + residual add + ReLU) with the
// constructor and overrides of FusedBatchNormalizationCudaCudnn<T>
// (include/nbla/cuda/cudnn/function/fused_batch_normalization.hpp).  Where the
// reference needs cuDNN's NHWC "Ex" path and otherwise falls back to a
// composite of three functions (cudnn/function/generic/
// fused_batch_normalization.cu:52-88), this class runs the fused kernels for
// every layout, both batch_stat modes and the three-output form.
#pragma once

#include <nbla/function/fused_batch_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class FusedBatchNormalizationHip : public FusedBatchNormalization<T> {
protected:
  int device_;
  Variable workspace_; // split-reduction partials + per-channel parameters
  size_t workspace_bytes_ = 0;

public:
  FusedBatchNormalizationHip(const Context &ctx, const vector<int> axes, float decay_rate,
                             float eps, bool batch_stat, const string &nonlinearity)
      : FusedBatchNormalization<T>(ctx, axes, decay_rate, eps, batch_stat, nonlinearity),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~FusedBatchNormalizationHip() {}
  virtual string name() { return "FusedBatchNormalizationHip"; }
  virtual vector<string> allowed_array_classes() {
    return SingletonManager::get<Hip>()->array_classes();
  }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs,
                             const vector<bool> &propagate_down, const vector<bool> &accum);
  void fused_batch_norm_forward(const Variables &inputs, const Variables &outputs,
                                const bool update_inputs);
};
} // namespace nbla
