// InstanceNormalizationHip<T>: host-side control flow of
// InstanceNormalizationCuda<T>
// (src/nbla/cuda/function/generic/instance_normalization.cu) over nblahip.
#include <nbla/hip/function/instance_normalization.hpp>
#include <nbla/variable.hpp>

#include <type_traits>

namespace nbla {

template <typename T>
void InstanceNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  InstanceNormalization<T>::setup_shapes(inputs, outputs);
  const auto x = inputs[0];
  // Channel-first and channel-last tensors are read in place; any other
  // position of the channel and batch axes goes through a device permutation
  // to channel-first and back, the counterpart of the ChannelFirstAdaptor the
  // reference uses (instance_normalization.cu:40-55,81-94,187-207).
  layout_.setup(x->shape(), this->batch_axis_, this->channel_axis_, x->shape()[this->channel_axis_]);
  channel_last_ = layout_.channel_last;
  channel_size_ = layout_.channels;
  batch_size_ = layout_.batch;
  spatial_size_ = layout_.spatial;
  // (as GroupNormalizationHip: ranges of samples per launch beyond 2^31 elements)
  NBLA_CHECK(channel_size_ * spatial_size_ < (Size_t(1) << 31) &&
                 (!layout_.data.needed() || x->size() < (Size_t(1) << 31)),
             error_code::value,
             "InstanceNormalizationHip indexes with 32 bits: fewer than 2^31 elements per sample "
             "required (per tensor where the layout needs a permutation).");
  mean_.reshape(Shape_t{batch_size_ * channel_size_}, true);
  var_.reshape(Shape_t{batch_size_ * channel_size_}, true);
  hip_set_device(this->device_); // argument errors above are reported without a device
  workspace_bytes_ =
      channel_last_ ? nblahip_in_cl_workspace_bytes(batch_size_, spatial_size_, channel_size_,
                                                    HipDtype<T>::code)
                    : nblahip_in_bwd_workspace_bytes(batch_size_, channel_size_, spatial_size_,
                                                     HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
  if (std::is_same<T, Half>::value) {
    const Size_t np = batch_size_ * channel_size_, ns = batch_size_ * channel_size_;
    stage_.reshape(Shape_t{ParamStage::capacity_for({np, np, np, np, ns, ns, ns, ns})}, true);
  }
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
  // (parameters and statistics a half graph stores in half are read and
  // written where they lie: ParamStage; statistics kept inside the function
  // stay float32)
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *beta = this->no_bias_ ? nullptr : st.in(inputs[this->beta_idx_]);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[this->gamma_idx_]);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const bool exposed = outputs.size() == 3;
  float *mean = exposed ? st.out(v_mean, false) : v_mean->cast_data_and_get_pointer<float>(this->ctx_, true);
  float *var = exposed ? st.out(v_var, false) : v_var->cast_data_and_get_pointer<float>(this->ctx_, true);
  st.load();
  const int bc_gamma = this->need_gamma_broadcast_ ? 1 : 0, bc_beta = this->need_beta_broadcast_ ? 1 : 0;
  if (channel_last_) {
    float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
    NBLA_HIP_CHECK(nblahip_in_cl_fwd(x, gamma, beta, y, mean, var, batch_size_, spatial_size_,
                                     channel_size_, bc_gamma, bc_beta, this->eps_,
                                     HipDtype<T>::code, ws, workspace_bytes_, nullptr));
    st.store();
    workspace_.data()->array()->clear();
    return;
  }
  const bool adapt = layout_.data.needed(), adapt_stats = layout_.stats.needed();
  const Size_t n = inputs[0]->size(), ns = batch_size_ * channel_size_;
  const T *xk = x;
  T *yk = y;
  float *mk = mean, *vk = var;
  if (adapt) {
    T *xs = adaptor_scratch<T>(adapt_a_, n, this->ctx_);
    layout_.data.to_kernel(x, xs, HipDtype<T>::code);
    xk = xs;
    yk = adaptor_scratch<T>(adapt_b_, n, this->ctx_);
  }
  if (adapt_stats) {
    // statistics and per-sample parameters are [batch..., channel] for the kernels
    mk = adaptor_scratch<float>(stat_a_, ns, this->ctx_);
    vk = adaptor_scratch<float>(stat_b_, ns, this->ctx_);
    if (gamma && !bc_gamma) {
      float *gk = adaptor_scratch<float>(stat_c_, ns, this->ctx_);
      layout_.stats.to_kernel(gamma, gk, NBLAHIP_F32);
      gamma = gk;
    }
    if (beta && !bc_beta) {
      float *bk = adaptor_scratch<float>(stat_d_, ns, this->ctx_);
      layout_.stats.to_kernel(beta, bk, NBLAHIP_F32);
      beta = bk;
    }
  }
  NBLA_HIP_CHECK(nblahip_in_fwd(xk, gamma, beta, yk, mk, vk, batch_size_, channel_size_,
                                spatial_size_, bc_gamma, bc_beta, this->eps_, HipDtype<T>::code,
                                nullptr));
  if (adapt) {
    layout_.data.to_caller(yk, y, false, HipDtype<T>::code);
    adaptor_release(adapt_a_);
    adaptor_release(adapt_b_);
  }
  if (adapt_stats) {
    layout_.stats.to_caller(mk, mean, false, NBLAHIP_F32);
    layout_.stats.to_caller(vk, var, false, NBLAHIP_F32);
    for (Variable *v : {&stat_a_, &stat_b_, &stat_c_, &stat_d_}) adaptor_release(*v);
  }
  st.store();
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
  }
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  ParamStage st;
  st.begin(this->ctx_, std::is_same<T, Half>::value, &stage_);
  const float *gamma = this->no_scale_ ? nullptr : st.in(inputs[gamma_idx]);
  if (outputs.size() == 3) {
    dmean = st.in(v_mean, true);
    dvar = st.in(v_var, true);
  }
  const float *mean = st.in(v_mean);
  const float *var = st.in(v_var);
  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *dbeta = !pd_beta ? nullptr : st.out(inputs[beta_idx], accum[beta_idx], true);
  float *dgamma = !pd_gamma ? nullptr : st.out(inputs[gamma_idx], accum[gamma_idx], true);
  st.load();
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  const int bc_gamma = this->need_gamma_broadcast_ ? 1 : 0, bc_beta = this->need_beta_broadcast_ ? 1 : 0;
  if (channel_last_) {
    NBLA_HIP_CHECK(nblahip_in_cl_bwd(x, dy, gamma, mean, var, dmean, dvar, dx, dgamma, dbeta,
                                     pd_x && accum[0], pd_gamma && accum[gamma_idx],
                                     pd_beta && accum[beta_idx], batch_size_, spatial_size_,
                                     channel_size_, bc_gamma, bc_beta, this->eps_,
                                     HipDtype<T>::code, ws, workspace_bytes_, nullptr));
    st.store();
    workspace_.data()->array()->clear();
    return;
  }
  const bool adapt = layout_.data.needed(), adapt_stats = layout_.stats.needed();
  const Size_t n = inputs[0]->size(), ns = batch_size_ * channel_size_;
  const T *xk = x, *dyk = dy;
  T *dxk = dx;
  if (adapt) {
    T *xs = adaptor_scratch<T>(adapt_a_, n, this->ctx_);
    T *dys = adaptor_scratch<T>(adapt_b_, n, this->ctx_);
    layout_.data.to_kernel(x, xs, HipDtype<T>::code);
    layout_.data.to_kernel(dy, dys, HipDtype<T>::code);
    xk = xs;
    dyk = dys;
    if (pd_x) dxk = adaptor_scratch<T>(adapt_c_, n, this->ctx_);
  }
  // Per-sample parameter gradients come back in the kernels' [batch...,
  // channel] order and are added to the caller's afterwards.
  float *dgk = dgamma, *dbk = dbeta;
  const bool own_dg = adapt_stats && dgamma && !bc_gamma, own_db = adapt_stats && dbeta && !bc_beta;
  if (adapt_stats) {
    float *mk = adaptor_scratch<float>(stat_a_, ns, this->ctx_);
    float *vk = adaptor_scratch<float>(stat_b_, ns, this->ctx_);
    layout_.stats.to_kernel(mean, mk, NBLAHIP_F32);
    layout_.stats.to_kernel(var, vk, NBLAHIP_F32);
    mean = mk;
    var = vk;
    if (dmean) {
      float *dmk = adaptor_scratch<float>(stat_c_, ns, this->ctx_);
      float *dvk = adaptor_scratch<float>(stat_d_, ns, this->ctx_);
      layout_.stats.to_kernel(dmean, dmk, NBLAHIP_F32);
      layout_.stats.to_kernel(dvar, dvk, NBLAHIP_F32);
      dmean = dmk;
      dvar = dvk;
    }
    if (gamma && !bc_gamma) {
      float *gk = adaptor_scratch<float>(stat_e_, ns, this->ctx_);
      layout_.stats.to_kernel(gamma, gk, NBLAHIP_F32);
      gamma = gk;
    }
    if (own_dg) dgk = adaptor_scratch<float>(stat_f_, ns, this->ctx_);
    if (own_db) dbk = adaptor_scratch<float>(stat_g_, ns, this->ctx_);
  }
  NBLA_HIP_CHECK(nblahip_in_bwd(xk, dyk, gamma, mean, var, dmean, dvar, dxk, dgk, dbk,
                                !adapt && pd_x && accum[0],
                                !own_dg && pd_gamma && accum[gamma_idx],
                                !own_db && pd_beta && accum[beta_idx], batch_size_, channel_size_,
                                spatial_size_, bc_gamma, bc_beta, this->eps_, HipDtype<T>::code, ws,
                                workspace_bytes_, nullptr));
  if (adapt) {
    if (pd_x) layout_.data.to_caller(dxk, dx, accum[0], HipDtype<T>::code);
    adaptor_release(adapt_a_);
    adaptor_release(adapt_b_);
    adaptor_release(adapt_c_);
  }
  if (adapt_stats) {
    if (own_dg) layout_.stats.to_caller(dgk, dgamma, accum[gamma_idx], NBLAHIP_F32);
    if (own_db) layout_.stats.to_caller(dbk, dbeta, accum[beta_idx], NBLAHIP_F32);
    for (Variable *v : {&stat_a_, &stat_b_, &stat_c_, &stat_d_, &stat_e_, &stat_f_, &stat_g_})
      adaptor_release(*v);
  }
  st.store();
  workspace_.data()->array()->clear();
}

template class InstanceNormalizationHip<float>;
template class InstanceNormalizationHip<Half>;
} // namespace nbla
