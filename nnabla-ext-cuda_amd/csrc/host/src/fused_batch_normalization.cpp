// FusedBatchNormalizationHip<T>: host-side control flow of
// FusedBatchNormalizationCudaCudnn<T> (src/nbla/cuda/cudnn/function/generic/
// fused_batch_normalization.cu) over the nblahip kernel layer.
#include <nbla/hip/function/fused_batch_normalization.hpp>
#include <nbla/variable.hpp>

namespace nbla {

template <typename T>
void FusedBatchNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  FusedBatchNormalization<T>::setup_impl(inputs, outputs);
  hip_set_device(this->device_);
  NBLA_CHECK(inputs[0]->size() < (Size_t(1) << 31), error_code::value,
             "FusedBatchNormalizationHip indexes with 32 bits: fewer than 2^31 elements "
             "required.");
  workspace_bytes_ = nblahip_bn_workspace_bytes(this->size0_, this->size1_, this->size2_,
                                                HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
}

template <typename T>
void FusedBatchNormalizationHip<T>::fused_batch_norm_forward(const Variables &inputs,
                                                             const Variables &outputs,
                                                             const bool update_inputs) {
  hip_set_device(this->device_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const float *beta = inputs[1]->template get_data_pointer<float>(this->ctx_);
  const float *gamma = inputs[2]->template get_data_pointer<float>(this->ctx_);
  const T *z = inputs.size() == 6 ? inputs[5]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  if (!this->batch_stat_) {
    const float *rm = inputs[3]->template get_data_pointer<float>(this->ctx_);
    const float *rv = inputs[4]->template get_data_pointer<float>(this->ctx_);
    NBLA_HIP_CHECK(nblahip_fused_bn_fwd_infer(x, z, rm, rv, gamma, beta, y, this->size0_,
                                              this->size1_, this->size2_, this->eps_,
                                              HipDtype<T>::code, nullptr));
    return;
  }
  Variable *batch_mean = &this->mean_;
  Variable *batch_var = &this->var_;
  if (outputs.size() == 3) {
    batch_mean = outputs[1];
    batch_var = outputs[2];
  }
  float *m = batch_mean->cast_data_and_get_pointer<float>(this->ctx_, true);
  float *v = batch_var->cast_data_and_get_pointer<float>(this->ctx_, true);
  // Running statistics are read-modify-write inputs; recompute leaves them.
  float *rm = !update_inputs ? nullptr
                             : inputs[3]->template cast_data_and_get_pointer<float>(this->ctx_);
  float *rv = !update_inputs ? nullptr
                             : inputs[4]->template cast_data_and_get_pointer<float>(this->ctx_);
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_fused_bn_fwd_train(x, z, gamma, beta, y, m, v, rm, rv, this->size0_,
                                            this->size1_, this->size2_, this->decay_rate_,
                                            this->eps_, HipDtype<T>::code, ws, workspace_bytes_,
                                            nullptr));
}

template <typename T>
void FusedBatchNormalizationHip<T>::forward_impl(const Variables &inputs,
                                                 const Variables &outputs) {
  fused_batch_norm_forward(inputs, outputs, true /* update_inputs */);
}

template <typename T>
void FusedBatchNormalizationHip<T>::recompute_impl(const Variables &inputs,
                                                   const Variables &outputs) {
  fused_batch_norm_forward(inputs, outputs, false /* update_inputs */);
}

template <typename T>
void FusedBatchNormalizationHip<T>::backward_impl(const Variables &inputs,
                                                  const Variables &outputs,
                                                  const vector<bool> &propagate_down,
                                                  const vector<bool> &accum) {
  hip_set_device(this->device_);
  const bool pd_x = propagate_down[0];
  const bool pd_beta = propagate_down[1];
  const bool pd_gamma = propagate_down[2];
  const bool pd_z = inputs.size() == 6 && propagate_down[5];
  if (!(pd_x || pd_beta || pd_gamma || pd_z)) return;

  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *y = outputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const float *gamma = inputs[2]->template get_data_pointer<float>(this->ctx_);
  const float *mean, *var, *dmean = nullptr, *dvar = nullptr;
  if (this->batch_stat_) {
    Variable *batch_mean = &this->mean_;
    Variable *batch_var = &this->var_;
    if (outputs.size() == 3) {
      batch_mean = outputs[1];
      batch_var = outputs[2];
      dmean = batch_mean->get_grad_pointer<float>(this->ctx_);
      dvar = batch_var->get_grad_pointer<float>(this->ctx_);
    }
    mean = batch_mean->get_data_pointer<float>(this->ctx_);
    var = batch_var->get_data_pointer<float>(this->ctx_);
  } else {
    mean = inputs[3]->template get_data_pointer<float>(this->ctx_);
    var = inputs[4]->template get_data_pointer<float>(this->ctx_);
  }
  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  T *dz = !pd_z ? nullptr : inputs[5]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[5]);
  float *dbeta =
      !pd_beta ? nullptr
               : inputs[1]->template cast_grad_and_get_pointer<float>(this->ctx_, !accum[1]);
  float *dgamma =
      !pd_gamma ? nullptr
                : inputs[2]->template cast_grad_and_get_pointer<float>(this->ctx_, !accum[2]);
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_fused_bn_bwd(
      x, y, dy, gamma, mean, var, dmean, dvar, dx, dz, dgamma, dbeta, pd_x && accum[0],
      pd_z && accum[5], pd_gamma && accum[2], pd_beta && accum[1], this->size0_, this->size1_,
      this->size2_, this->eps_, this->batch_stat_ ? 1 : 0, HipDtype<T>::code, ws,
      workspace_bytes_, nullptr));
}

template class FusedBatchNormalizationHip<float>;
template class FusedBatchNormalizationHip<Half>;
} // namespace nbla
