// BatchNormalizationHip<T>: host-side control flow of the reference's
// BatchNormalizationCuda<T> (src/nbla/cuda/function/generic/batch_normalization.cu)
// over the nblahip kernel layer.
#include <nbla/hip/function/batch_normalization.hpp>
#include <nbla/variable.hpp>

#include <type_traits>

namespace nbla {

template <typename T>
void BatchNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  BatchNormalization<T>::setup_impl(inputs, outputs);
  hip_set_device(this->device_);
  // Tensors of 2^31 elements and more run in ranges along the outermost axes
  // (local statistics, merge, normalization per range inside the kernel
  // layer); one slice of those axes must stay below that.
  NBLA_CHECK(this->size1_ * this->size2_ < (Size_t(1) << 31), error_code::value,
             "BatchNormalizationHip indexes with 32 bits: fewer than 2^31 elements per slice of the "
             "axes ahead of the channel axis required.");
  workspace_bytes_ = nblahip_bn_workspace_bytes(this->size0_, this->size1_, this->size2_,
                                                HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
  if (std::is_same<T, Half>::value) {
    const Size_t c = this->size1_;
    stage_.reshape(Shape_t{ParamStage::capacity_for({c, c, c, c, c, c, c, c})}, true);
  }
}

template <typename T>
void BatchNormalizationHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  if (this->batch_stat_) { // Training mode.
    forward_impl_batch(inputs, outputs, true /* update_inputs */);
  } else { // Testing mode.
    forward_impl_global(inputs, outputs);
  }
}

template <typename T>
void BatchNormalizationHip<T>::recompute_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  if (this->batch_stat_) {
    forward_impl_batch(inputs, outputs, false /* update_inputs */);
  } else {
    forward_impl_global(inputs, outputs);
  }
}

template <typename T>
void BatchNormalizationHip<T>::forward_impl_batch(const Variables &inputs, const Variables &outputs,
                                                  const bool update_inputs) {
  // Batch statistics go to the outputs when they are exposed, otherwise to
  // the members backward reads them from.
  Variable *batch_mean = &this->mean_;
  Variable *batch_var = &this->var_;
  if (outputs.size() == 3) {
    batch_mean = outputs[1];
    batch_var = outputs[2];
  }
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  // (parameters and statistics a half graph stores in half are read and
  // written where they lie: ParamStage)
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *beta = this->no_bias_ ? nullptr : st.in(inputs[this->b_idx_]);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[this->g_idx_]);
  // Running statistics are read-modify-write inputs; recompute leaves them.
  float *rm = !update_inputs ? nullptr : st.out(inputs[this->m_idx_], true);
  float *rv = !update_inputs ? nullptr : st.out(inputs[this->v_idx_], true);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  // (statistics kept inside the function stay float32; exposed ones follow the parameters)
  const bool exposed = outputs.size() == 3;
  float *m = exposed ? st.out(batch_mean, false)
                     : batch_mean->cast_data_and_get_pointer<float>(this->ctx_, true);
  float *v = exposed ? st.out(batch_var, false)
                     : batch_var->cast_data_and_get_pointer<float>(this->ctx_, true);
  st.load();
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_bn_fwd_train(x, gamma, beta, y, m, v, rm, rv, this->size0_, this->size1_,
                                      this->size2_, this->decay_rate_, this->eps_,
                                      HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  st.store();
}

template <typename T>
void BatchNormalizationHip<T>::forward_impl_global(const Variables &inputs,
                                                   const Variables &outputs) {
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *beta = this->no_bias_ ? nullptr : st.in(inputs[this->b_idx_]);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[this->g_idx_]);
  const float *rm = st.in(inputs[this->m_idx_]);
  const float *rv = st.in(inputs[this->v_idx_]);
  st.load();
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_bn_fwd_infer(x, rm, rv, gamma, beta, y, this->size0_, this->size1_,
                                      this->size2_, this->eps_, HipDtype<T>::code, nullptr));
}

template <typename T>
void BatchNormalizationHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                             const vector<bool> &propagate_down,
                                             const vector<bool> &accum) {
  hip_set_device(this->device_);
  if (this->batch_stat_) { // Training mode.
    backward_impl_batch(inputs, outputs, propagate_down, accum);
  } else { // Testing mode.
    backward_impl_global(inputs, outputs, propagate_down, accum);
  }
}

template <typename T>
void BatchNormalizationHip<T>::backward_impl_batch(const Variables &inputs,
                                                   const Variables &outputs,
                                                   const vector<bool> &propagate_down,
                                                   const vector<bool> &accum) {
  backward_launch(inputs, outputs, propagate_down, accum, true);
}

template <typename T>
void BatchNormalizationHip<T>::backward_impl_global(const Variables &inputs,
                                                    const Variables &outputs,
                                                    const vector<bool> &propagate_down,
                                                    const vector<bool> &accum) {
  backward_launch(inputs, outputs, propagate_down, accum, false);
}

template <typename T>
void BatchNormalizationHip<T>::backward_launch(const Variables &inputs, const Variables &outputs,
                                               const vector<bool> &propagate_down,
                                               const vector<bool> &accum, bool batch_stat) {
  const bool pd_x = propagate_down[0];
  const bool pd_beta = !this->no_bias_ && propagate_down[this->b_idx_];
  const bool pd_gamma = !this->no_scale_ && propagate_down[this->g_idx_];
  if (!(pd_x || pd_beta || pd_gamma)) return;

  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[this->g_idx_]);

  // Statistics the forward normalised with, and the gradients that reach the
  // mean/var outputs in the three-output form.
  const float *mean, *var, *dmean = nullptr, *dvar = nullptr;
  if (batch_stat) {
    Variable *batch_mean = &this->mean_;
    Variable *batch_var = &this->var_;
    if (outputs.size() == 3) {
      batch_mean = outputs[1];
      batch_var = outputs[2];
      dmean = st.in(batch_mean, true);
      dvar = st.in(batch_var, true);
    }
    mean = st.in(batch_mean);
    var = st.in(batch_var);
  } else {
    mean = st.in(inputs[this->m_idx_]);
    var = st.in(inputs[this->v_idx_]);
  }

  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *dbeta = !pd_beta ? nullptr : st.out(inputs[this->b_idx_], accum[this->b_idx_], true);
  float *dgamma = !pd_gamma ? nullptr : st.out(inputs[this->g_idx_], accum[this->g_idx_], true);
  st.load();
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_bn_bwd(
      x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta, pd_x && accum[0],
      pd_gamma && accum[this->g_idx_], pd_beta && accum[this->b_idx_], this->size0_, this->size1_,
      this->size2_, this->eps_, batch_stat ? 1 : 0, HipDtype<T>::code, ws, workspace_bytes_,
      nullptr));
  st.store();
}

template class BatchNormalizationHip<float>;
template class BatchNormalizationHip<Half>;
} // namespace nbla
