// TensorNormalizationHip<T> and WeightStandardizationHip<T>: the reference's
// TensorNormalizationCuda<T> / WeightStandardizationCuda<T>
// (src/nbla/cuda/function/generic/tensor_normalization.cu:22-46,
// weight_standardization.cu:22-46) set the device and call the core's
// composites; here both run on the batch-statistics BatchNormalization entry
// points of nblahip (no running statistics; no transposes when the kept axes
// are adjacent).
#include <nbla/hip/function/tensor_normalization.hpp>
#include <nbla/hip/function/weight_standardization.hpp>
#include <nbla/variable.hpp>

namespace nbla {

namespace {

// Shared forward: x viewed as [size0, size1, size2], statistics per index of
// size1; through `adaptor` (when needed) for kept axes that are not adjacent.
template <typename T> struct NormView {
  Size_t size0, size1, size2;
  float eps;
  size_t ws_bytes;

  void forward(const Context &ctx, Variable *x_v, Variable *beta_v, Variable *gamma_v,
               Variable *y_v, Variable *mean_v, Variable *var_v, Variable &ws_v,
               const AxisAdaptor *adaptor = nullptr, Variable *buf_a = nullptr,
               Variable *buf_b = nullptr) const {
    const T *x = x_v->get_data_pointer<T>(ctx);
    const float *beta = beta_v ? beta_v->get_data_pointer<float>(ctx) : nullptr;
    const float *gamma = gamma_v ? gamma_v->get_data_pointer<float>(ctx) : nullptr;
    T *y = y_v->cast_data_and_get_pointer<T>(ctx, true);
    float *m = mean_v->cast_data_and_get_pointer<float>(ctx, true);
    float *v = var_v->cast_data_and_get_pointer<float>(ctx, true);
    float *ws = ws_v.cast_data_and_get_pointer<float>(ctx, true);
    const bool adapt = adaptor && adaptor->needed();
    T *yk = y;
    if (adapt) {
      T *xs = adaptor_scratch<T>(*buf_a, x_v->size(), ctx);
      adaptor->to_kernel(x, xs, HipDtype<T>::code);
      x = xs;
      yk = adaptor_scratch<T>(*buf_b, x_v->size(), ctx);
    }
    NBLA_HIP_CHECK(nblahip_bn_fwd_train(x, gamma, beta, yk, m, v, nullptr, nullptr, size0, size1,
                                        size2, 0.f, eps, HipDtype<T>::code, ws, ws_bytes, nullptr));
    if (adapt) {
      adaptor->to_caller(yk, y, false, HipDtype<T>::code);
      adaptor_release(*buf_a);
      adaptor_release(*buf_b);
    }
    ws_v.data()->array()->clear();
  }
};

} // namespace

// Adjacent kept axes are the "channel" extent of the [size0, C, size2] view of
// the tensor as it lies in memory.  Any other set is gathered behind the
// remaining axes by a device permutation ([others..., kept...], i.e. the
// channel-last view [size0, C, 1]) and y / dx are permuted back; the core's
// composite the reference calls transposes for such sets as well
// (tensor_normalization.cu:22-46).  The kept axes keep their order, so beta,
// gamma and the statistics are read and written as the caller lays them out.
static void view_of_axes(const Shape_t &shape, const vector<int> &sorted_axes, Size_t &s0,
                         Size_t &s1, Size_t &s2, AxisAdaptor *adaptor = nullptr) {
  bool adjacent = true;
  for (size_t i = 1; i < sorted_axes.size(); ++i)
    adjacent = adjacent && sorted_axes[i] == sorted_axes[i - 1] + 1;
  s0 = s1 = s2 = 1;
  if (!adjacent) {
    NBLA_CHECK(adaptor != nullptr, error_code::value, "axes must be adjacent.");
    adaptor->setup(shape, sorted_axes, true);
    for (int i = 0; i < static_cast<int>(shape.size()); ++i) {
      const bool kept = std::find(sorted_axes.begin(), sorted_axes.end(), i) != sorted_axes.end();
      (kept ? s1 : s0) *= shape[i];
    }
    return;
  }
  if (adaptor) adaptor->setup(Shape_t{1}, vector<int>{0}); // not needed
  const int first = sorted_axes.front(), last = sorted_axes.back();
  for (int i = 0; i < static_cast<int>(shape.size()); ++i) {
    if (i < first) s0 *= shape[i];
    else if (i <= last) s1 *= shape[i];
    else s2 *= shape[i];
  }
}

template <typename T>
void TensorNormalizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  TensorNormalization<T>::setup_shapes(inputs, outputs);
  view_of_axes(inputs[0]->shape(), this->axes_, size0_, size1_, size2_, &adaptor_);
  NBLA_CHECK(inputs[0]->size() < (Size_t(1) << 31), error_code::value,
             "TensorNormalizationHip indexes with 32 bits: fewer than 2^31 elements required.");
  mean_.reshape(Shape_t{size1_}, true);
  var_.reshape(Shape_t{size1_}, true);
  hip_set_device(this->device_); // argument errors above are reported without a device
  workspace_bytes_ = nblahip_bn_workspace_bytes(size0_, size1_, size2_, HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
}

template <typename T>
void TensorNormalizationHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  const bool three = outputs.size() == 3;
  const NormView<T> view{size0_, size1_, size2_, this->eps_, workspace_bytes_};
  view.forward(this->ctx_, inputs[0], this->no_bias_ ? nullptr : inputs[this->beta_idx_],
               this->no_scale_ ? nullptr : inputs[this->gamma_idx_], outputs[0],
               three ? outputs[1] : &mean_, three ? outputs[2] : &var_, workspace_, &adaptor_,
               &adapt_a_, &adapt_b_);
}

template <typename T>
void TensorNormalizationHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                              const vector<bool> &propagate_down,
                                              const vector<bool> &accum) {
  const bool pd_x = propagate_down[0];
  const bool pd_beta = !this->no_bias_ && propagate_down[this->beta_idx_];
  const bool pd_gamma = !this->no_scale_ && propagate_down[this->gamma_idx_];
  if (!(pd_x || pd_beta || pd_gamma)) return;
  hip_set_device(this->device_);
  const bool three = outputs.size() == 3;
  Variable *mean_v = three ? outputs[1] : &mean_;
  Variable *var_v = three ? outputs[2] : &var_;
  const float *dmean = three ? mean_v->get_grad_pointer<float>(this->ctx_) : nullptr;
  const float *dvar = three ? var_v->get_grad_pointer<float>(this->ctx_) : nullptr;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const float *gamma = this->no_scale_ ? nullptr
                                       : inputs[this->gamma_idx_]->template get_data_pointer<float>(this->ctx_);
  const float *mean = mean_v->get_data_pointer<float>(this->ctx_);
  const float *var = var_v->get_data_pointer<float>(this->ctx_);
  T *dx = !pd_x ? nullptr : inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *dbeta = !pd_beta ? nullptr
                          : inputs[this->beta_idx_]->template cast_grad_and_get_pointer<float>(
                                this->ctx_, !accum[this->beta_idx_]);
  float *dgamma = !pd_gamma ? nullptr
                            : inputs[this->gamma_idx_]->template cast_grad_and_get_pointer<float>(
                                  this->ctx_, !accum[this->gamma_idx_]);
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
  NBLA_HIP_CHECK(nblahip_bn_bwd(x, dy, gamma, mean, var, dmean, dvar, dxk, dgamma, dbeta,
                                !adapt && pd_x && accum[0], pd_gamma && accum[this->gamma_idx_],
                                pd_beta && accum[this->beta_idx_], size0_, size1_, size2_,
                                this->eps_, 1, HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  if (adapt) {
    if (pd_x) adaptor_.to_caller(dxk, dx, accum[0], HipDtype<T>::code);
    adaptor_release(adapt_a_);
    adaptor_release(adapt_b_);
    adaptor_release(adapt_c_);
  }
  workspace_.data()->array()->clear();
}

template <typename T>
void WeightStandardizationHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  WeightStandardization<T>::setup_shapes(inputs, outputs);
  view_of_axes(inputs[0]->shape(), vector<int>{this->channel_axis_}, size0_, size1_, size2_);
  NBLA_CHECK(inputs[0]->size() < (Size_t(1) << 31), error_code::value,
             "WeightStandardizationHip indexes with 32 bits: fewer than 2^31 elements required.");
  mean_.reshape(Shape_t{size1_}, true);
  var_.reshape(Shape_t{size1_}, true);
  hip_set_device(this->device_);
  workspace_bytes_ = nblahip_bn_workspace_bytes(size0_, size1_, size2_, HipDtype<T>::code);
  workspace_.reshape(Shape_t{static_cast<Size_t>((workspace_bytes_ + 3) / 4)}, true);
}

template <typename T>
void WeightStandardizationHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->device_);
  const bool three = outputs.size() == 3;
  const NormView<T> view{size0_, size1_, size2_, this->eps_, workspace_bytes_};
  view.forward(this->ctx_, inputs[0], nullptr, nullptr, outputs[0], three ? outputs[1] : &mean_,
               three ? outputs[2] : &var_, workspace_);
}

template <typename T>
void WeightStandardizationHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                                const vector<bool> &propagate_down,
                                                const vector<bool> &accum) {
  if (!propagate_down[0]) return;
  hip_set_device(this->device_);
  const bool three = outputs.size() == 3;
  Variable *mean_v = three ? outputs[1] : &mean_;
  Variable *var_v = three ? outputs[2] : &var_;
  const float *dmean = three ? mean_v->get_grad_pointer<float>(this->ctx_) : nullptr;
  const float *dvar = three ? var_v->get_grad_pointer<float>(this->ctx_) : nullptr;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const float *mean = mean_v->get_data_pointer<float>(this->ctx_);
  const float *var = var_v->get_data_pointer<float>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  float *ws = workspace_.cast_data_and_get_pointer<float>(this->ctx_, true);
  NBLA_HIP_CHECK(nblahip_bn_bwd(x, dy, nullptr, mean, var, dmean, dvar, dx, nullptr, nullptr,
                                accum[0], 0, 0, size0_, size1_, size2_, this->eps_, 1,
                                HipDtype<T>::code, ws, workspace_bytes_, nullptr));
  workspace_.data()->array()->clear();
}

template class TensorNormalizationHip<float>;
template class TensorNormalizationHip<Half>;
template class WeightStandardizationHip<float>;
template class WeightStandardizationHip<Half>;
} // namespace nbla
