// LayerNormalizationHip<T>: host-side control flow of LayerNormalizationCuda<T>
// (src/nbla/cuda/function/generic/layer_normalization.cu) over nblahip.
#include <nbla/hip/function/layer_normalization.hpp>
#include <nbla/variable.hpp>

#include <type_traits>

namespace nbla {

template <typename T>
void LayerNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  LayerNormalization<T>::setup_shapes(inputs, outputs);
  const auto x_shape = inputs[0]->shape();
  // The kernels reduce over trailing axes.  Batch axes that are not the
  // leading ones are brought to the front by a device permutation, and y / dx
  // are permuted back (the reference hands such layouts to the core's
  // function instead, layer_normalization.cu:43-51).  The non-batch axes keep
  // their order, so beta and gamma are read as they are, and the statistics
  // come out in batch-axis order, as the caller lays them out.
  vector<int> ba(this->batch_axis_);
  std::sort(ba.begin(), ba.end());
  adaptor_.setup(x_shape, ba);
  batch_size_ = 1;
  for (const auto b : ba) batch_size_ *= x_shape[b];
  reduce_size_ = inputs[0]->size() / std::max<Size_t>(batch_size_, 1);
  // Tensors of 2^31 elements and more run as several launches over ranges of
  // rows (the kernel layer indexes one launch with 32 bits); one row, and a
  // tensor that has to be permuted first, must stay below that.
  NBLA_CHECK(reduce_size_ < (Size_t(1) << 31) &&
                 (!adaptor_.needed() || inputs[0]->size() < (Size_t(1) << 31)),
             error_code::value,
             "LayerNormalizationHip indexes with 32 bits: fewer than 2^31 elements per row "
             "required (per tensor where the batch axes are not the leading ones).");
  mean_.reshape(Shape_t{batch_size_}, true);
  var_.reshape(Shape_t{batch_size_}, true);
  hip_set_device(this->device_); // argument errors above are reported without a device
  workspace_bytes_ = nblahip_ln_bwd_workspace_bytes(batch_size_, reduce_size_, HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
  if (std::is_same<T, Half>::value) {
    stage_.reshape(Shape_t{ParamStage::capacity_for({reduce_size_, reduce_size_, reduce_size_,
                                                     reduce_size_, batch_size_, batch_size_,
                                                     batch_size_, batch_size_})},
                   true);
  }
}

template <typename T>
void LayerNormalizationHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  Variable *v_mean = &mean_;
  Variable *v_var = &var_;
  if (outputs.size() == 3) { // statistics are exposed
    v_mean = outputs[1];
    v_var = outputs[2];
  }
  const int beta_idx = 1;
  const int gamma_idx = this->no_bias_ ? 1 : 2;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *beta = this->no_bias_ ? nullptr : st.in(inputs[beta_idx]);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[gamma_idx]);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  // (statistics kept inside the function stay float32; exposed ones follow the parameters)
  const bool exposed = outputs.size() == 3;
  float *mean = exposed ? st.out(v_mean, false) : v_mean->cast_data_and_get_pointer<float>(this->ctx_, true);
  float *var = exposed ? st.out(v_var, false) : v_var->cast_data_and_get_pointer<float>(this->ctx_, true);
  st.load();
  const T *xk = x;
  T *yk = y;
  if (adaptor_.needed()) {
    const Size_t n = inputs[0]->size();
    T *xs = adaptor_scratch<T>(adapt_a_, n, this->ctx_);
    adaptor_.to_kernel(x, xs, HipDtype<T>::code);
    xk = xs;
    yk = adaptor_scratch<T>(adapt_b_, n, this->ctx_);
  }
  NBLA_HIP_CHECK(nblahip_ln_fwd(xk, gamma, beta, yk, mean, var, batch_size_, reduce_size_,
                                this->eps_, HipDtype<T>::code, nullptr));
  st.store();
  if (adaptor_.needed()) {
    adaptor_.to_caller(yk, y, false, HipDtype<T>::code);
    adaptor_release(adapt_a_);
    adaptor_release(adapt_b_);
  }
}

template <typename T>
void LayerNormalizationHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                             const vector<bool> &propagate_down,
                                             const vector<bool> &accum) {
  hip_set_device(this->device_);
  const int beta_idx = 1;
  const int gamma_idx = this->no_bias_ ? 1 : 2;
  const bool pd_x = propagate_down[0];
  const bool pd_beta = !this->no_bias_ && propagate_down[beta_idx];
  const bool pd_gamma = !this->no_scale_ && propagate_down[gamma_idx];
  if (!(pd_x || pd_beta || pd_gamma)) return;

  Variable *v_mean = &mean_;
  Variable *v_var = &var_;
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[gamma_idx]);
  const float *dmean = nullptr, *dvar = nullptr;
  if (outputs.size() == 3) {
    v_mean = outputs[1];
    v_var = outputs[2];
    dmean = st.in(v_mean, true);
    dvar = st.in(v_var, true);
  }
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const float *mean = st.in(v_mean);
  const float *var = st.in(v_var);
  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *dbeta = !pd_beta ? nullptr : st.out(inputs[beta_idx], accum[beta_idx], true);
  float *dgamma = !pd_gamma ? nullptr : st.out(inputs[gamma_idx], accum[gamma_idx], true);
  st.load();
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  const bool adapt = adaptor_.needed();
  T *dxk = dx;
  if (adapt) {
    const Size_t n = inputs[0]->size();
    T *xs = adaptor_scratch<T>(adapt_a_, n, this->ctx_);
    T *dys = adaptor_scratch<T>(adapt_b_, n, this->ctx_);
    adaptor_.to_kernel(x, xs, HipDtype<T>::code);
    adaptor_.to_kernel(dy, dys, HipDtype<T>::code);
    x = xs;
    dy = dys;
    if (pd_x) dxk = adaptor_scratch<T>(adapt_c_, n, this->ctx_);
  }
  NBLA_HIP_CHECK(nblahip_ln_bwd(x, dy, gamma, mean, var, dmean, dvar, dxk, dgamma, dbeta,
                                !adapt && pd_x && accum[0], pd_gamma && accum[gamma_idx],
                                pd_beta && accum[beta_idx], batch_size_, reduce_size_, this->eps_,
                                HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  st.store();
  if (adapt) {
    if (pd_x) adaptor_.to_caller(dxk, dx, accum[0], HipDtype<T>::code);
    adaptor_release(adapt_a_);
    adaptor_release(adapt_b_);
    adaptor_release(adapt_c_);
  }
  // Scratch is only needed inside the call (the reference clears its buffers
  // the same way, layer_normalization.cu:202-203,236-237).
  workspace_.data()->array()->clear();
}

template class LayerNormalizationHip<float>;
template class LayerNormalizationHip<Half>;
} // namespace nbla
