// InstanceNormalizationHip<T>: host-side control flow of
// InstanceNormalizationCuda<T>
// (src/nbla/cuda/function/generic/instance_normalization.cu) over nblahip.
#include <nbla/hip/function/instance_normalization.hpp>
#include <nbla/variable.hpp>

namespace nbla {

template <typename T>
void InstanceNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  InstanceNormalization<T>::setup_shapes(inputs, outputs);
  const auto x = inputs[0];
  const int c = this->channel_axis_;
  // Two layouts run without a transpose: channel-first (the channel axis
  // right after the leading batch axes) and channel-last (batch axes leading,
  // channel axis last).  The reference brings every other layout to
  // channel-first through the core's ChannelFirstAdaptor
  // (instance_normalization.cu:40-55); that adaptor is not part of this backend.
  const int nb = static_cast<int>(this->batch_axis_.size());
  const int ndim = static_cast<int>(x->shape().size());
  bool batch_leading = true;
  for (int b : this->batch_axis_) batch_leading = batch_leading && b < nb;
  const bool channel_first = batch_leading && c == nb;
  channel_last_ = batch_leading && !channel_first && c == ndim - 1;
  NBLA_CHECK(channel_first || channel_last_, error_code::not_implemented,
             "InstanceNormalizationHip supports batch axes leading with the channel axis right "
             "after them (channel-first) or last (channel-last).");
  channel_size_ = x->shape()[c];
  batch_size_ = 1;
  for (int b : this->batch_axis_) batch_size_ *= x->shape()[b];
  spatial_size_ = (batch_size_ > 0 && channel_size_ > 0) ? x->size() / (batch_size_ * channel_size_) : 0;
  NBLA_CHECK(x->size() < (Size_t(1) << 31), error_code::value,
             "InstanceNormalizationHip indexes with 32 bits: fewer than 2^31 elements required.");
  mean_.reshape(Shape_t{batch_size_ * channel_size_}, true);
  var_.reshape(Shape_t{batch_size_ * channel_size_}, true);
  hip_set_device(this->device_); // argument errors above are reported without a device
  workspace_bytes_ =
      channel_last_ ? nblahip_in_cl_workspace_bytes(batch_size_, spatial_size_, channel_size_,
                                                    HipDtype<T>::code)
                    : nblahip_in_bwd_workspace_bytes(batch_size_, channel_size_, spatial_size_,
                                                     HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
}

template <typename T>
void InstanceNormalizationHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  Variable *v_mean = &mean_;
  Variable *v_var = &var_;
  if (outputs.size() == 3) {
    v_mean = outputs[1];
    v_var = outputs[2];
  }
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const float *beta = this->no_bias_ ? nullptr
                                     : inputs[this->beta_idx_]->template get_data_pointer<float>(this->ctx_);
  const float *gamma = this->no_scale_ ? nullptr
                                       : inputs[this->gamma_idx_]->template get_data_pointer<float>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  float *mean = v_mean->cast_data_and_get_pointer<float>(this->ctx_, true);
  float *var = v_var->cast_data_and_get_pointer<float>(this->ctx_, true);
  if (channel_last_) {
    float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
    NBLA_HIP_CHECK(nblahip_in_cl_fwd(x, gamma, beta, y, mean, var, batch_size_, spatial_size_,
                                     channel_size_, this->need_gamma_broadcast_ ? 1 : 0,
                                     this->need_beta_broadcast_ ? 1 : 0, this->eps_,
                                     HipDtype<T>::code, ws, workspace_bytes_, nullptr));
    workspace_.data()->array()->clear();
    return;
  }
  NBLA_HIP_CHECK(nblahip_in_fwd(x, gamma, beta, y, mean, var, batch_size_, channel_size_,
                                spatial_size_, this->need_gamma_broadcast_ ? 1 : 0,
                                this->need_beta_broadcast_ ? 1 : 0, this->eps_, HipDtype<T>::code,
                                nullptr));
}

template <typename T>
void InstanceNormalizationHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                                const vector<bool> &propagate_down,
                                                const vector<bool> &accum) {
  hip_set_device(this->device_);
  const int beta_idx = this->beta_idx_;
  const int gamma_idx = this->gamma_idx_;
  const bool pd_x = propagate_down[0];
  const bool pd_beta = !this->no_bias_ && propagate_down[beta_idx];
  const bool pd_gamma = !this->no_scale_ && propagate_down[gamma_idx];
  if (!(pd_x || pd_beta || pd_gamma)) return;

  Variable *v_mean = &mean_;
  Variable *v_var = &var_;
  const float *dmean = nullptr, *dvar = nullptr;
  if (outputs.size() == 3) {
    v_mean = outputs[1];
    v_var = outputs[2];
    dmean = v_mean->get_grad_pointer<float>(this->ctx_);
    dvar = v_var->get_grad_pointer<float>(this->ctx_);
  }
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const float *gamma =
      this->no_scale_ ? nullptr : inputs[gamma_idx]->template get_data_pointer<float>(this->ctx_);
  const float *mean = v_mean->get_data_pointer<float>(this->ctx_);
  const float *var = v_var->get_data_pointer<float>(this->ctx_);
  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *dbeta = !pd_beta ? nullptr
                          : inputs[beta_idx]->template cast_grad_and_get_pointer<float>(
                                this->ctx_, !accum[beta_idx]);
  float *dgamma = !pd_gamma ? nullptr
                            : inputs[gamma_idx]->template cast_grad_and_get_pointer<float>(
                                  this->ctx_, !accum[gamma_idx]);
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  if (channel_last_) {
    NBLA_HIP_CHECK(nblahip_in_cl_bwd(x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta,
                                     pd_x && accum[0], pd_gamma && accum[gamma_idx],
                                     pd_beta && accum[beta_idx], batch_size_, spatial_size_,
                                     channel_size_, this->need_gamma_broadcast_ ? 1 : 0,
                                     this->need_beta_broadcast_ ? 1 : 0, this->eps_,
                                     HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  } else {
    NBLA_HIP_CHECK(nblahip_in_bwd(x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta,
                                  pd_x && accum[0], pd_gamma && accum[gamma_idx],
                                  pd_beta && accum[beta_idx], batch_size_, channel_size_,
                                  spatial_size_, this->need_gamma_broadcast_ ? 1 : 0,
                                  this->need_beta_broadcast_ ? 1 : 0, this->eps_,
                                  HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  }
  workspace_.data()->array()->clear();
}

template class InstanceNormalizationHip<float>;
template class InstanceNormalizationHip<Half>;
} // namespace nbla
