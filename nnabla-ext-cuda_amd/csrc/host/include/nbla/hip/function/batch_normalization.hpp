// BatchNormalizationHip<T>: the "hip" implementation of BatchNormalization,
// same constructor, name()/allowed_array_classes() and *_impl overrides as
// BatchNormalizationCuda<T> (include/nbla/cuda/function/batch_normalization.hpp:31-85).
// The kernels take statistics, gamma/beta and their gradients as float32 for
// every T, as the reference's cudnn context does
// (src/nbla/cuda/cudnn/function/generic/batch_normalization.cu:94-99,193-227).
// Arrays that a "hip:half" graph stores in half - the plain cuda:half config's
// Tc (batch_normalization.cu:124-143) - are read and written where they lie
// and keep their type (nbla/hip/utils/param_stage.hpp); the batch statistics
// the function keeps for its own backward stay float32.
#pragma once

#include <nbla/function/batch_normalization.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/utils/param_stage.hpp>

namespace nbla {

template <typename T> class BatchNormalizationHip : public BatchNormalization<T> {
protected:
  int device_;
  Variable workspace_; // split-reduction partials + per-channel parameters
  size_t workspace_bytes_ = 0;
  Variable stage_; // float32 staging of parameters / statistics stored in half (ParamStage)

public:
  BatchNormalizationHip(const Context &ctx, const vector<int> axes, float decay_rate, float eps,
                        bool batch_stat, bool no_scale, bool no_bias)
      : BatchNormalization<T>(ctx, axes, decay_rate, eps, batch_stat, no_scale, no_bias),
        device_(std::stoi(ctx.device_id)) {}
  virtual ~BatchNormalizationHip() {}
  virtual string name() { return "BatchNormalizationHip"; }
  virtual vector<string> allowed_array_classes() {
    return SingletonManager::get<Hip>()->array_classes();
  }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs,
                             const vector<bool> &propagate_down, const vector<bool> &accum);
  virtual void forward_impl_batch(const Variables &inputs, const Variables &outputs,
                                  const bool update_inputs);
  virtual void forward_impl_global(const Variables &inputs, const Variables &outputs);
  // backward_impl dispatches on batch_stat to one of these two, as the
  // reference does (batch_normalization.cu:200-212); a subclass may override
  // either (the reference's cudnn class overrides backward_impl_batch,
  // include/nbla/cuda/cudnn/function/batch_normalization.hpp:90).  The
  // reference leaves the inference-mode backward to the core's
  // backward_impl_global on the CPU; here it runs on the device.
  virtual void backward_impl_batch(const Variables &inputs, const Variables &outputs,
                                   const vector<bool> &propagate_down, const vector<bool> &accum);
  virtual void backward_impl_global(const Variables &inputs, const Variables &outputs,
                                    const vector<bool> &propagate_down, const vector<bool> &accum);
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs);

private:
  void backward_launch(const Variables &inputs, const Variables &outputs,
                       const vector<bool> &propagate_down, const vector<bool> &accum,
                       bool batch_stat);
};
} // namespace nbla
