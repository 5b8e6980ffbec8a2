// forward_impl of the "hip:float" Function classes: fetch device pointers through the Variable interface, obtain
// scratch from the backend's caching allocator, call the kernel library.
#include <nbla/hip/common.hpp>
#include <nbla/hip/function/arithmetic.hpp>
#include <nbla/hip/function/binary.hpp>
#include <nbla/hip/function/inq.hpp>
#include <nbla/hip/function/quantize.hpp>
#include <nbla/hip/function/quantize_linear.hpp>
#include <nbla/hip/function/range_recorder.hpp>
#include <nbla/random_manager.hpp>

#include <algorithm>
#include <random>

namespace nbla {

NBLA_REGISTER_FUNCTION_SOURCE(RangeRecorder, int, double, bool);

namespace {
vector<int64_t> to_i64(const Shape_t &s) { return vector<int64_t>(s.begin(), s.end()); }
} // namespace

// ---------------------------------------------------------------- quantizers
template <typename T>
void FixedPointQuantizeHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  NBLA_HIP_CALL(nbla_hip_fixed_point_quantize_f32(x, y, (size_t)inputs[0]->size(), this->sign_, this->n_, this->delta_,
                                                  nullptr));
}

template <typename T> void Pow2QuantizeHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  NBLA_HIP_CALL(nbla_hip_pow2_quantize_f32(x, y, (size_t)inputs[0]->size(), this->sign_, this->with_zero_, this->n_,
                                           this->m_, nullptr));
}

// min_max_quantize.cpp:45-127: the shape checks; none of the helper functions the CPU class creates is needed.
template <typename T> void MinMaxQuantizeHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  auto x = inputs[0];
  auto qr_min = inputs[1], qr_max = inputs[2], ql_min = inputs[3], ql_max = inputs[4];
  NBLA_CHECK(ql_min->ndim() == ql_max->ndim() && ql_max->ndim() == qr_min->ndim() && qr_min->ndim() == qr_max->ndim(),
             error_code::value, "All input dimensions must be same.");
  NBLA_CHECK(ql_min->shape() == ql_max->shape() && ql_max->shape() == qr_min->shape() &&
                 qr_min->shape() == qr_max->shape(),
             error_code::value, "All shapes among ql_min, ql_max, qr_min, and qr_max must be same.");
  NBLA_CHECK(x->ndim() == ql_min->ndim(), error_code::value, "x and ql_min must have the same number of dimensions.");
  for (Size_t i = 0; i < ql_min->ndim(); i++) {
    NBLA_CHECK(ql_min->shape()[i] == 1 || x->shape()[i] == ql_min->shape()[i], error_code::value,
               "x.shape and ql_min.shape must be same except for i-th dimension where ql_min.shape[i] == 1.");
  }
  outputs[0]->reshape(x->shape(), true);
  this->scale_sptr_ = make_shared<Variable>(ql_min->shape());
}

template <typename T> void MinMaxQuantizeHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const vector<int64_t> xshape = to_i64(inputs[0]->shape()), qshape = to_i64(inputs[1]->shape());
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  // qr_min / qr_max are running state: updated in place, as the reference updates its parameters
  T *qr_min = inputs[1]->cast_data_and_get_pointer<T>(this->ctx_);
  T *qr_max = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_);
  const T *ql_min = inputs[3]->get_data_pointer<T>(this->ctx_);
  const T *ql_max = inputs[4]->get_data_pointer<T>(this->ctx_);
  T *scale = this->scale_sptr_->template cast_data_and_get_pointer<T>(this->ctx_, true);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_min_max_quantize_workspace_bytes(xshape.data(), (int)xshape.size(), qshape.data()),
                  this->ctx_);
  NBLA_HIP_CALL(nbla_hip_min_max_quantize_f32(x, y, xshape.data(), (int)xshape.size(), qshape.data(), qr_min, qr_max,
                                              ql_min, ql_max, scale, this->decay_, this->x_min_max_, this->ema_,
                                              this->eps_, ws.pointer(), ws.bytes(), nullptr));
}

// fixed_point_quantize.cpp:103-127
template <typename T>
void FixedPointQuantizeHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                             const vector<bool> &propagate_down, const vector<bool> &accum) {
  if (!propagate_down[0])
    return;
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  NBLA_HIP_CALL(nbla_hip_fixed_point_quantize_backward_f32(dy, x, dx, (size_t)inputs[0]->size(), this->sign_, this->n_,
                                                           this->delta_, this->ste_fine_grained_, accum[0], nullptr));
}

// pow2_quantize.cpp:127-156
template <typename T>
void Pow2QuantizeHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                       const vector<bool> &propagate_down, const vector<bool> &accum) {
  if (!propagate_down[0])
    return;
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  NBLA_HIP_CALL(nbla_hip_pow2_quantize_backward_f32(dy, x, dx, (size_t)inputs[0]->size(), this->sign_,
                                                    this->with_zero_, this->n_, this->m_, this->ste_fine_grained_,
                                                    accum[0], nullptr));
}

// min_max_quantize.cpp:225-350
template <typename T>
void MinMaxQuantizeHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                         const vector<bool> &propagate_down, const vector<bool> &accum) {
  NBLA_CHECK(!(propagate_down[3] || propagate_down[4]), error_code::value,
             "Backward to x(inputs[0]), qr_min(inputs[1]), and/or qr_max(inputs[2])are only allowed.");
  if (!(propagate_down[0] || propagate_down[1] || propagate_down[2]))
    return;
  hip_set_device(this->ctx_);
  const vector<int64_t> xshape = to_i64(inputs[0]->shape()), qshape = to_i64(inputs[1]->shape());
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *qr_min = inputs[1]->get_data_pointer<T>(this->ctx_);
  const T *qr_max = inputs[2]->get_data_pointer<T>(this->ctx_);
  const T *ql_min = inputs[3]->get_data_pointer<T>(this->ctx_);
  const T *ql_max = inputs[4]->get_data_pointer<T>(this->ctx_);
  const T *scale = this->scale_sptr_->template get_data_pointer<T>(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const bool range = !(this->x_min_max_ || this->ema_);
  T *dx = propagate_down[0] ? inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]) : nullptr;
  T *g_min = (range && propagate_down[1]) ? inputs[1]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[1]) : nullptr;
  T *g_max = (range && propagate_down[2]) ? inputs[2]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[2]) : nullptr;
  HipWorkspace ws(nbla_hip_min_max_quantize_backward_workspace_bytes(xshape.data(), (int)xshape.size(), qshape.data()),
                  this->ctx_);
  NBLA_HIP_CALL(nbla_hip_min_max_quantize_backward_f32(
      dy, x, dx, xshape.data(), (int)xshape.size(), qshape.data(), qr_min, qr_max, ql_min, ql_max, scale, g_min, g_max,
      this->ste_fine_grained_, this->x_min_max_, this->ema_, accum[0], accum[1], accum[2], ws.pointer(), ws.bytes(),
      nullptr));
}

// ------------------------------------------------------------- binary affine
// binary_weight_affine.cpp:32-72
template <typename T> void BinaryWeightAffineHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_affine_shapes(this->base_axis_, inputs[0], inputs[1], inputs.size() == 5 ? inputs[4] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  this->w_row_ = shapes_.w_row;
  this->w_col_ = shapes_.w_col;
  NBLA_CHECK(inputs[1]->shape() == inputs[2]->shape(), error_code::value,
             "Binary and float weights must have same size.");
  NBLA_CHECK(inputs[3]->size() == shapes_.w_col, error_code::value, "Size of alpha must be equal to output size.");
  outputs[0]->reshape(shapes_.out_shape, true);
}

// binary_connect_affine.cpp:29-57
template <typename T> void BinaryConnectAffineHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_affine_shapes(this->base_axis_, inputs[0], inputs[1], inputs.size() == 4 ? inputs[3] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  NBLA_CHECK(inputs[1]->shape() == inputs[2]->shape(), error_code::value,
             "Binary and float weights must have same size.");
  outputs[0]->reshape(shapes_.out_shape, true);
}

template <typename T>
void BinaryWeightAffineHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const AffineShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *wb = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_, true);
  T *alpha = inputs[3]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const T *b = inputs.size() == 5 ? inputs[4]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_binary_affine_workspace_bytes(s.i_row, s.i_col, s.w_col), this->ctx_);
  NBLA_HIP_CALL(nbla_hip_binary_weight_affine_f32(x, w, wb, alpha, b, y, s.i_row, s.i_col, s.w_col,
                                                  this->quantize_zero_to_, ws.pointer(), ws.bytes(), nullptr));
}

template <typename T>
void BinaryConnectAffineHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const AffineShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *wb = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const T *b = inputs.size() == 4 ? inputs[3]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_binary_affine_workspace_bytes(s.i_row, s.i_col, s.w_col), this->ctx_);
  NBLA_HIP_CALL(nbla_hip_binary_connect_affine_f32(x, w, wb, b, y, s.i_row, s.i_col, s.w_col, this->quantize_zero_to_,
                                                   ws.pointer(), ws.bytes(), nullptr));
}

namespace {
// Shared body of the affine backward passes: `bias_index` is the position of the bias among the inputs (or -1).
template <typename T, typename Call>
void affine_backward_common(const Context &ctx, const AffineShapes &s, const Variables &inputs, const Variables &outputs,
                            const vector<bool> &propagate_down, const vector<bool> &accum, int bias_index, Call call) {
  const bool has_bias = bias_index >= 0 && (int)inputs.size() > bias_index;
  const bool pb = has_bias && propagate_down[bias_index];
  if (!(propagate_down[0] || propagate_down[1] || pb))
    return;
  hip_set_device(ctx);
  const T *x = inputs[0]->get_data_pointer<T>(ctx);
  const T *dy = outputs[0]->get_grad_pointer<T>(ctx);
  T *dx = propagate_down[0] ? inputs[0]->cast_grad_and_get_pointer<T>(ctx, !accum[0]) : nullptr;
  T *dw = propagate_down[1] ? inputs[1]->cast_grad_and_get_pointer<T>(ctx, !accum[1]) : nullptr;
  T *db = pb ? inputs[bias_index]->cast_grad_and_get_pointer<T>(ctx, !accum[bias_index]) : nullptr;
  HipWorkspace ws(nbla_hip_affine_backward_workspace_bytes(s.i_row, s.i_col, s.w_col), ctx);
  call(dy, x, dx, dw, db, (int)accum[0], (int)accum[1], has_bias ? (int)accum[bias_index] : 0, ws);
}
} // namespace

// binary_weight_affine.cpp:124-146
template <typename T>
void BinaryWeightAffineHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                             const vector<bool> &propagate_down, const vector<bool> &accum) {
  const AffineShapes &s = shapes_;
  affine_backward_common<T>(this->ctx_, s, inputs, outputs, propagate_down, accum, 4,
                            [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
                              const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
                              const T *wb = inputs[2]->get_data_pointer<T>(this->ctx_);
                              const T *alpha = inputs[3]->get_data_pointer<T>(this->ctx_);
                              NBLA_HIP_CALL(nbla_hip_binary_affine_backward_f32(
                                  dy, x, w, wb, alpha, dx, dw, db, s.i_row, s.i_col, s.w_col, this->quantize_zero_to_,
                                  ax, aw, ab, ws.pointer(), ws.bytes(), nullptr));
                            });
}

// binary_connect_affine.cpp:73-92
template <typename T>
void BinaryConnectAffineHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                              const vector<bool> &propagate_down, const vector<bool> &accum) {
  const AffineShapes &s = shapes_;
  affine_backward_common<T>(this->ctx_, s, inputs, outputs, propagate_down, accum, 3,
                            [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
                              const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
                              const T *wb = inputs[2]->get_data_pointer<T>(this->ctx_);
                              NBLA_HIP_CALL(nbla_hip_binary_affine_backward_f32(
                                  dy, x, w, wb, nullptr, dx, dw, db, s.i_row, s.i_col, s.w_col,
                                  this->quantize_zero_to_, ax, aw, ab, ws.pointer(), ws.bytes(), nullptr));
                            });
}

// -------------------------------------------------------- binary convolution
// binary_weight_convolution.cpp:33-70
template <typename T>
void BinaryWeightConvolutionHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_conv_shapes(this->base_axis_, this->pad_, this->stride_, this->dilation_, this->group_, inputs[0],
                              inputs[1], inputs.size() == 5 ? inputs[4] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  this->channels_o_ = (int)shapes_.channels_o;
  this->col_w_ = (int)shapes_.inner_size_k;
  NBLA_CHECK(inputs[1]->shape() == inputs[2]->shape(), error_code::value,
             "Binary and float weights must have same size.");
  NBLA_CHECK(inputs[3]->size() == shapes_.channels_o, error_code::value,
             "Size of alpha must be equal to the number of output channels.");
  outputs[0]->reshape(shapes_.out_shape, true);
}

// binary_connect_convolution.cpp:35-65
template <typename T>
void BinaryConnectConvolutionHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_conv_shapes(this->base_axis_, this->pad_, this->stride_, this->dilation_, this->group_, inputs[0],
                              inputs[1], inputs.size() == 4 ? inputs[3] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  NBLA_CHECK(inputs[1]->shape() == inputs[2]->shape(), error_code::value,
             "Binary and float weights must have same size.");
  outputs[0]->reshape(shapes_.out_shape, true);
}

template <typename T>
void BinaryWeightConvolutionHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const ConvShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *wb = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_, true);
  T *alpha = inputs[3]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const T *b = inputs.size() == 5 ? inputs[4]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_binary_convolution_workspace_bytes(
                      s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o, s.kernel.data(),
                      s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_),
                  this->ctx_);
  NBLA_HIP_CALL(nbla_hip_binary_weight_convolution_f32(
      x, w, wb, alpha, b, y, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o, s.kernel.data(),
      s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_, ws.pointer(), ws.bytes(),
      nullptr));
}

template <typename T>
void BinaryConnectConvolutionHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const ConvShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *wb = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const T *b = inputs.size() == 4 ? inputs[3]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_binary_convolution_workspace_bytes(
                      s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o, s.kernel.data(),
                      s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_),
                  this->ctx_);
  NBLA_HIP_CALL(nbla_hip_binary_connect_convolution_f32(
      x, w, wb, b, y, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o, s.kernel.data(),
      s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_, ws.pointer(), ws.bytes(),
      nullptr));
}

namespace {
// Shared body of the convolution backward passes: `bias_index` is the position of the bias among the inputs.
template <typename T, typename Call>
void conv_backward_common(const Context &ctx, const ConvShapes &s, const Variables &inputs, const Variables &outputs,
                          const vector<bool> &propagate_down, const vector<bool> &accum, int bias_index, Call call) {
  const bool has_bias = (int)inputs.size() > bias_index;
  const bool pb = has_bias && propagate_down[bias_index];
  if (!(propagate_down[0] || propagate_down[1] || pb))
    return;
  hip_set_device(ctx);
  const T *x = inputs[0]->get_data_pointer<T>(ctx);
  const T *dy = outputs[0]->get_grad_pointer<T>(ctx);
  T *dx = propagate_down[0] ? inputs[0]->cast_grad_and_get_pointer<T>(ctx, !accum[0]) : nullptr;
  T *dw = propagate_down[1] ? inputs[1]->cast_grad_and_get_pointer<T>(ctx, !accum[1]) : nullptr;
  T *db = pb ? inputs[bias_index]->cast_grad_and_get_pointer<T>(ctx, !accum[bias_index]) : nullptr;
  HipWorkspace ws(nbla_hip_convolution_backward_workspace_bytes(s.outer, s.channels_i, s.spatial_dims,
                                                                s.spatial_i.data(), s.channels_o, s.kernel.data(),
                                                                s.pad.data(), s.stride.data(), s.dilation.data(),
                                                                s.group),
                  ctx);
  call(dy, x, dx, dw, db, (int)accum[0], (int)accum[1], has_bias ? (int)accum[bias_index] : 0, ws);
}
} // namespace

// binary_weight_convolution.cpp:119-142
template <typename T>
void BinaryWeightConvolutionHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                                  const vector<bool> &propagate_down, const vector<bool> &accum) {
  const ConvShapes &s = shapes_;
  conv_backward_common<T>(
      this->ctx_, s, inputs, outputs, propagate_down, accum, 4,
      [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
        const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
        const T *wb = inputs[2]->get_data_pointer<T>(this->ctx_);
        const T *alpha = inputs[3]->get_data_pointer<T>(this->ctx_);
        NBLA_HIP_CALL(nbla_hip_binary_convolution_backward_f32(
            dy, x, w, wb, alpha, dx, dw, db, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o,
            s.kernel.data(), s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_, ax, aw,
            ab, ws.pointer(), ws.bytes(), nullptr));
      });
}

// binary_connect_convolution.cpp:83-103
template <typename T>
void BinaryConnectConvolutionHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                                   const vector<bool> &propagate_down, const vector<bool> &accum) {
  const ConvShapes &s = shapes_;
  conv_backward_common<T>(
      this->ctx_, s, inputs, outputs, propagate_down, accum, 3,
      [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
        const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
        const T *wb = inputs[2]->get_data_pointer<T>(this->ctx_);
        NBLA_HIP_CALL(nbla_hip_binary_convolution_backward_f32(
            dy, x, w, wb, nullptr, dx, dw, db, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o,
            s.kernel.data(), s.pad.data(), s.stride.data(), s.dilation.data(), s.group, this->quantize_zero_to_, ax, aw,
            ab, ws.pointer(), ws.bytes(), nullptr));
      });
}

// ----------------------------------------------------------------------- INQ
namespace {
// Steps A, B, D and F of INQAffine<T, T1>::setup_impl (inq_affine.cpp:34-79; the same in inq_convolution.cpp:35-102):
// indicator shape, selection algorithm, the generator of the "random" selection, counter and snapshots.
void inq_setup_state(Variable *weights, Variable *indicators, const string &selection_algorithm, int seed,
                     std::mt19937 &rgen, std::bernoulli_distribution &rdist, int &minibatch_counter,
                     Variable &old_weights, Variable &old_indicators) {
  NBLA_CHECK(weights->shape().size() == indicators->shape().size(), error_code::value,
             "Indicators and weights must have same size. Ndim of weights: %d != ndim of indicators: %d.",
             (int)weights->shape().size(), (int)indicators->shape().size());
  NBLA_CHECK(weights->shape() == indicators->shape(), error_code::value,
             "Indicators and weights must have same size.");
  NBLA_CHECK(selection_algorithm == "largest_abs" || selection_algorithm == "random", error_code::value,
             "Provided value for selection algorithm not valid: %s. Valid values are \"largest_abs\" and \"random\".",
             selection_algorithm.c_str());
  if (selection_algorithm == "random") {
    std::random_device rdev;
    rgen = std::mt19937(seed == -1 ? rdev() : (unsigned)seed);
    rdist = std::bernoulli_distribution(0.5);
  }
  minibatch_counter = 0;
  old_weights.reshape(weights->shape(), true);
  old_indicators.reshape(weights->shape(), true);
  old_indicators.data()->zero();
}

// The indicator update the current minibatch calls for (inq_affine.cpp:104-113): 0 none, 1 fix all, 2 largest_abs,
// 3 random.
int inq_current_step(const vector<int> &inq_iterations, int minibatch_counter, const string &selection_algorithm) {
  if (std::find(inq_iterations.begin(), inq_iterations.end(), minibatch_counter) == inq_iterations.end())
    return 0;
  if (inq_iterations.back() == minibatch_counter)
    return 1;
  return selection_algorithm == "largest_abs" ? 2 : 3;
}

// The Bernoulli stream of inq_affine.cpp:84-86,147: rdist_(rgen), one draw per learnable weight, from the
// process-wide generator when the seed is -1.
struct InqDraw {
  std::mt19937 *gen;
  std::bernoulli_distribution *dist;
};
void draw_bernoulli(void *ctx, uint8_t *out, int64_t count) {
  InqDraw *d = static_cast<InqDraw *>(ctx);
  for (int64_t i = 0; i < count; ++i)
    out[i] = (*d->dist)(*d->gen) ? 1 : 0;
}
} // namespace

// inq_affine.cpp:34-79
template <typename T, typename T1>
void INQAffineHip<T, T1>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_affine_shapes(this->base_axis_, inputs[0], inputs[1], inputs.size() == 4 ? inputs[3] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  outputs[0]->reshape(shapes_.out_shape, true);
  inq_setup_state(inputs[1], inputs[2], this->selection_algorithm_, this->seed_, this->rgen_, this->rdist_,
                  this->minibatch_counter_, this->old_weights_, this->old_indicators_);
}

// inq_convolution.cpp:35-102
template <typename T, typename T1>
void INQConvolutionHip<T, T1>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_conv_shapes(this->base_axis_, this->pad_, this->stride_, this->dilation_, this->group_, inputs[0],
                              inputs[1], inputs.size() == 4 ? inputs[3] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  outputs[0]->reshape(shapes_.out_shape, true);
  inq_setup_state(inputs[1], inputs[2], this->selection_algorithm_, this->seed_, this->rgen_, this->rdist_,
                  this->minibatch_counter_, this->old_weights_, this->old_indicators_);
}

template <typename T, typename T1>
void INQAffineHip<T, T1>::run(const Variables &inputs, const Variables &outputs, int step) {
  hip_set_device(this->ctx_);
  const AffineShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *w = inputs[1]->cast_data_and_get_pointer<T>(this->ctx_);
  T1 *ind = inputs[2]->cast_data_and_get_pointer<T1>(this->ctx_);
  T *old_w = this->old_weights_.template cast_data_and_get_pointer<T>(this->ctx_);
  T1 *old_i = this->old_indicators_.template cast_data_and_get_pointer<T1>(this->ctx_);
  const T *b = inputs.size() == 4 ? inputs[3]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_inq_affine_workspace_bytes(s.i_row, s.i_col, s.w_col, step), this->ctx_);
  InqDraw draw{this->seed_ == -1 ? &SingletonManager::get<RandomManager>()->get_rand_generator() : &this->rgen_,
               &this->rdist_};
  NBLA_HIP_CALL(nbla_hip_inq_affine_f32(x, w, ind, old_w, old_i, b, y, s.i_row, s.i_col, s.w_col, this->num_bits_,
                                        step, draw_bernoulli, &draw, ws.pointer(), ws.bytes(), nullptr));
}
template <typename T, typename T1>
void INQAffineHip<T, T1>::forward_impl(const Variables &inputs, const Variables &outputs) {
  run(inputs, outputs,
      inq_current_step(this->inq_iterations_, this->minibatch_counter_, this->selection_algorithm_));
  this->minibatch_counter_++; // inq_affine.cpp:200
}
template <typename T, typename T1>
void INQAffineHip<T, T1>::recompute_impl(const Variables &inputs, const Variables &outputs) {
  run(inputs, outputs, -1); // inq_affine.cpp:208-216: the product alone
}

template <typename T, typename T1>
void INQConvolutionHip<T, T1>::run(const Variables &inputs, const Variables &outputs, int step) {
  hip_set_device(this->ctx_);
  const ConvShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *w = inputs[1]->cast_data_and_get_pointer<T>(this->ctx_);
  T1 *ind = inputs[2]->cast_data_and_get_pointer<T1>(this->ctx_);
  T *old_w = this->old_weights_.template cast_data_and_get_pointer<T>(this->ctx_);
  T1 *old_i = this->old_indicators_.template cast_data_and_get_pointer<T1>(this->ctx_);
  const T *b = inputs.size() == 4 ? inputs[3]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_inq_convolution_workspace_bytes(s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(),
                                                           s.channels_o, s.kernel.data(), s.pad.data(),
                                                           s.stride.data(), s.dilation.data(), s.group, step),
                  this->ctx_);
  InqDraw draw{this->seed_ == -1 ? &SingletonManager::get<RandomManager>()->get_rand_generator() : &this->rgen_,
               &this->rdist_};
  NBLA_HIP_CALL(nbla_hip_inq_convolution_f32(x, w, ind, old_w, old_i, b, y, s.outer, s.channels_i, s.spatial_dims,
                                             s.spatial_i.data(), s.channels_o, s.kernel.data(), s.pad.data(),
                                             s.stride.data(), s.dilation.data(), s.group, this->num_bits_, step,
                                             draw_bernoulli, &draw, ws.pointer(), ws.bytes(), nullptr));
}
template <typename T, typename T1>
void INQConvolutionHip<T, T1>::forward_impl(const Variables &inputs, const Variables &outputs) {
  run(inputs, outputs,
      inq_current_step(this->inq_iterations_, this->minibatch_counter_, this->selection_algorithm_));
  this->minibatch_counter_++;
}
template <typename T, typename T1>
void INQConvolutionHip<T, T1>::recompute_impl(const Variables &inputs, const Variables &outputs) {
  run(inputs, outputs, -1);
}

// ------------------------------------------------------------ Affine and ReLU
// affine.cpp:29-78
template <typename T> void AffineHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  shapes_ = infer_affine_shapes(this->base_axis_, inputs[0], inputs[1], inputs.size() == 3 ? inputs[2] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  this->i_row_ = shapes_.i_row;
  this->i_col_ = shapes_.i_col;
  this->w_row_ = shapes_.w_row;
  this->w_col_ = shapes_.w_col;
  this->o_row_ = shapes_.i_row;
  this->o_col_ = shapes_.w_col;
  outputs[0]->reshape(shapes_.out_shape, true);
}

// convolution.cpp:41-160
template <typename T> void ConvolutionHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  NBLA_CHECK(!this->channel_last_, error_code::not_implemented,
             "The passed argument channel_last_=true is not supported in Convolution.");
  shapes_ = infer_conv_shapes(this->base_axis_, this->pad_, this->stride_, this->dilation_, this->group_, inputs[0],
                              inputs[1], inputs.size() == 3 ? inputs[2] : nullptr);
  this->base_axis_ = shapes_.base_axis;
  this->channels_i_ = shapes_.channels_i;
  this->channels_o_ = shapes_.channels_o;
  this->channels_g_ = shapes_.channels_g;
  this->spatial_dims_ = shapes_.spatial_dims;
  this->outer_size_ = shapes_.outer;
  this->inner_size_k_ = shapes_.inner_size_k;
  outputs[0]->reshape(shapes_.out_shape, true);
}

template <typename T> void AffineHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const AffineShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  const T *b = inputs.size() == 3 ? inputs[2]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_affine_workspace_bytes(s.i_row, s.i_col, s.w_col), this->ctx_);
  NBLA_HIP_CALL(nbla_hip_affine_digits_f32(x, w, b, y, s.i_row, s.i_col, s.w_col, ws.pointer(), ws.bytes(), nullptr));
}

// inq_affine.cpp:218-232: Affine backward with the (quantized) weights
template <typename T, typename T1>
void INQAffineHip<T, T1>::backward_impl(const Variables &inputs, const Variables &outputs,
                                        const vector<bool> &propagate_down, const vector<bool> &accum) {
  const AffineShapes &s = shapes_;
  affine_backward_common<T>(this->ctx_, s, inputs, outputs, propagate_down, accum, 3,
                            [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
                              const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
                              NBLA_HIP_CALL(nbla_hip_affine_backward_f32(dy, x, w, dx, dw, db, s.i_row, s.i_col, s.w_col,
                                                                         ax, aw, ab, ws.pointer(), ws.bytes(), nullptr));
                            });
}

// inq_convolution.cpp:220-232
template <typename T, typename T1>
void INQConvolutionHip<T, T1>::backward_impl(const Variables &inputs, const Variables &outputs,
                                             const vector<bool> &propagate_down, const vector<bool> &accum) {
  const ConvShapes &s = shapes_;
  conv_backward_common<T>(
      this->ctx_, s, inputs, outputs, propagate_down, accum, 3,
      [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
        const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
        NBLA_HIP_CALL(nbla_hip_convolution_backward_f32(
            dy, x, w, dx, dw, db, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o,
            s.kernel.data(), s.pad.data(), s.stride.data(), s.dilation.data(), s.group, ax, aw, ab, ws.pointer(),
            ws.bytes(), nullptr));
      });
}

// convolution.cpp:161-197
template <typename T> void ConvolutionHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const ConvShapes &s = shapes_;
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
  const T *b = inputs.size() == 3 ? inputs[2]->get_data_pointer<T>(this->ctx_) : nullptr;
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_convolution_workspace_bytes(s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(),
                                                       s.channels_o, s.kernel.data(), s.pad.data(), s.stride.data(),
                                                       s.dilation.data(), s.group),
                  this->ctx_);
  NBLA_HIP_CALL(nbla_hip_convolution_f32(x, w, b, y, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(),
                                         s.channels_o, s.kernel.data(), s.pad.data(), s.stride.data(),
                                         s.dilation.data(), s.group, ws.pointer(), ws.bytes(), nullptr));
}

// convolution.cpp:199-283
template <typename T>
void ConvolutionHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                      const vector<bool> &propagate_down, const vector<bool> &accum) {
  const ConvShapes &s = shapes_;
  conv_backward_common<T>(
      this->ctx_, s, inputs, outputs, propagate_down, accum, 2,
      [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
        const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
        NBLA_HIP_CALL(nbla_hip_convolution_backward_f32(
            dy, x, w, dx, dw, db, s.outer, s.channels_i, s.spatial_dims, s.spatial_i.data(), s.channels_o,
            s.kernel.data(), s.pad.data(), s.stride.data(), s.dilation.data(), s.group, ax, aw, ab, ws.pointer(),
            ws.bytes(), nullptr));
      });
}

// affine.cpp:98-140
template <typename T>
void AffineHip<T>::backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                                 const vector<bool> &accum) {
  const AffineShapes &s = shapes_;
  affine_backward_common<T>(this->ctx_, s, inputs, outputs, propagate_down, accum, 2,
                            [&](const T *dy, const T *x, T *dx, T *dw, T *db, int ax, int aw, int ab, HipWorkspace &ws) {
                              const T *w = inputs[1]->get_data_pointer<T>(this->ctx_);
                              NBLA_HIP_CALL(nbla_hip_affine_backward_f32(dy, x, w, dx, dw, db, s.i_row, s.i_col, s.w_col,
                                                                         ax, aw, ab, ws.pointer(), ws.bytes(), nullptr));
                            });
}

// relu.cpp:51-66
template <typename T>
void ReLUHip<T>::backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                               const vector<bool> &accum) {
  if (!propagate_down[0])
    return;
  hip_set_device(this->ctx_);
  const T *y = outputs[0]->get_data_pointer<T>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  NBLA_HIP_CALL(nbla_hip_relu_backward_f32(dy, y, dx, (size_t)inputs[0]->size(), accum[0], nullptr));
}

template <typename T> void ReLUHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  NBLA_HIP_CALL(nbla_hip_relu_f32(x, y, (size_t)inputs[0]->size(), nullptr));
}

// ------------------------------------------------------------ Add2 and Concatenate
namespace {
vector<int64_t> shape64(const Variable *v) {
  const Shape_t s = v->shape();
  return vector<int64_t>(s.begin(), s.end());
}
} // namespace

// add2.cpp:39-47; inputs of different shapes: the BcAdd2 fall-back of :28-37 (utils/base_transform_binary.hpp:339-356)
template <typename T> void Add2Hip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x0 = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *x1 = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  if (inputs[0]->shape() == inputs[1]->shape()) {
    NBLA_HIP_CALL(nbla_hip_add2_f32(x0, x1, y, (size_t)inputs[0]->size(), nullptr));
    return;
  }
  const vector<int64_t> s0 = shape64(inputs[0]), s1 = shape64(inputs[1]);
  NBLA_HIP_CALL(nbla_hip_broadcast2_f32(NBLA_HIP_BINARY2_ADD, x0, s0.data(), x1, s1.data(), y, (int)s0.size(), nullptr));
}

// add2.cpp:59-77
template <typename T>
void Add2Hip<T>::backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                               const vector<bool> &accum) {
  if (!(propagate_down[0] || propagate_down[1]))
    return;
  hip_set_device(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  const bool same = inputs[0]->shape() == inputs[1]->shape();
  const vector<int64_t> s0 = shape64(inputs[0]), s1 = shape64(inputs[1]);
  for (int i = 0; i < 2; ++i) {
    if (!propagate_down[i])
      continue;
    T *dx = inputs[i]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[i]);
    if (same)
      NBLA_HIP_CALL(nbla_hip_add2_backward_f32(dy, dx, (size_t)inputs[0]->size(), accum[i], nullptr));
    else { // utils/base_transform_binary.hpp:358-392
      HipWorkspace ws(nbla_hip_broadcast2_backward_workspace_bytes(i, s0.data(), s1.data(), (int)s0.size()), this->ctx_);
      NBLA_HIP_CALL(nbla_hip_broadcast2_backward_f32(NBLA_HIP_BINARY2_ADD, i, dy, nullptr, s0.data(), nullptr, s1.data(),
                                                     dx, (int)s0.size(), accum[i], ws.pointer(), ws.bytes(), nullptr));
    }
  }
}

// Sub2, Mul2, Div2, Pow2: utils/base_transform_binary.hpp:339-400 with the expressions of sub2.hpp:41, mul2.hpp:42,
// div2.hpp:44, pow2.hpp:44-47; inputs of one shape take the plain element-wise kernels, others the broadcasting ones
#define NBLA_HIP_DEFINE_BINARY2(NAME, OP)                                                                              \
  template <typename T> void NAME##Hip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {           \
    hip_set_device(this->ctx_);                                                                                        \
    const T *x0 = inputs[0]->get_data_pointer<T>(this->ctx_);                                                          \
    const T *x1 = inputs[1]->get_data_pointer<T>(this->ctx_);                                                          \
    T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);                                                 \
    if (OP != NBLA_HIP_BINARY2_POW && inputs[0]->shape() == inputs[1]->shape()) {                                      \
      NBLA_HIP_CALL(nbla_hip_binary2_f32(OP, x0, x1, y, (size_t)inputs[0]->size(), nullptr));                          \
      return;                                                                                                          \
    }                                                                                                                  \
    const vector<int64_t> s0 = shape64(inputs[0]), s1 = shape64(inputs[1]);                                            \
    NBLA_HIP_CALL(nbla_hip_broadcast2_f32(OP, x0, s0.data(), x1, s1.data(), y, (int)s0.size(), nullptr));              \
  }                                                                                                                    \
  template <typename T>                                                                                                \
  void NAME##Hip<T>::backward_impl(const Variables &inputs, const Variables &outputs,                                  \
                                   const vector<bool> &propagate_down, const vector<bool> &accum) {                   \
    if (!(propagate_down[0] || propagate_down[1]))                                                                     \
      return;                                                                                                          \
    hip_set_device(this->ctx_);                                                                                        \
    const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);                                                         \
    const T *x0 = inputs[0]->get_data_pointer<T>(this->ctx_);                                                          \
    const T *x1 = inputs[1]->get_data_pointer<T>(this->ctx_);                                                          \
    const bool same = inputs[0]->shape() == inputs[1]->shape();                                                        \
    const vector<int64_t> s0 = shape64(inputs[0]), s1 = shape64(inputs[1]);                                            \
    for (int i = 0; i < 2; ++i) {                                                                                      \
      if (!propagate_down[i])                                                                                          \
        continue;                                                                                                      \
      T *dx = inputs[i]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[i]);                                          \
      if (OP != NBLA_HIP_BINARY2_POW && same)                                                                          \
        NBLA_HIP_CALL(nbla_hip_binary2_backward_f32(OP, i, dy, x0, x1, dx, (size_t)inputs[0]->size(), accum[i],        \
                                                    nullptr));                                                         \
      else {                                                                                                           \
        HipWorkspace ws(nbla_hip_broadcast2_backward_workspace_bytes(i, s0.data(), s1.data(), (int)s0.size()),         \
                        this->ctx_);                                                                                   \
        NBLA_HIP_CALL(nbla_hip_broadcast2_backward_f32(OP, i, dy, x0, s0.data(), x1, s1.data(), dx, (int)s0.size(),    \
                                                       accum[i], ws.pointer(), ws.bytes(), nullptr));                  \
      }                                                                                                                \
    }                                                                                                                  \
  }
NBLA_HIP_DEFINE_BINARY2(Sub2, NBLA_HIP_BINARY2_SUB)
NBLA_HIP_DEFINE_BINARY2(Mul2, NBLA_HIP_BINARY2_MUL)
NBLA_HIP_DEFINE_BINARY2(Div2, NBLA_HIP_BINARY2_DIV)
NBLA_HIP_DEFINE_BINARY2(Pow2, NBLA_HIP_BINARY2_POW) // pow2.hpp:44-47
#undef NBLA_HIP_DEFINE_BINARY2

// concatenate.cpp:62-76
template <typename T> void ConcatenateHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  int64_t inner_offset = 0;
  for (Variables::size_type c = 0; c < inputs.size(); ++c) {
    const T *x = inputs[c]->get_data_pointer<T>(this->ctx_);
    const int64_t inner_size = inputs[c]->size(this->axis_);
    NBLA_HIP_CALL(nbla_hip_copy_rows_f32(x, inner_size, y + inner_offset, this->inner_total_size_, this->outer_size_,
                                         inner_size, 0, nullptr));
    inner_offset += inner_size;
  }
}

// concatenate.cpp:78-104
template <typename T>
void ConcatenateHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                      const vector<bool> &propagate_down, const vector<bool> &accum) {
  hip_set_device(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  int64_t inner_offset = 0;
  for (Variables::size_type c = 0; c < inputs.size(); ++c) {
    const int64_t inner_size = inputs[c]->size(this->axis_);
    if (propagate_down[c]) {
      T *dx = inputs[c]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[c]);
      NBLA_HIP_CALL(nbla_hip_copy_rows_f32(dy + inner_offset, this->inner_total_size_, dx, inner_size,
                                           this->outer_size_, inner_size, accum[c], nullptr));
    }
    inner_offset += inner_size;
  }
}

// ------------------------------------------- QuantizeLinear / DequantizeLinear / Prune

// quantize_linear.cpp:28-46 and dequantize_linear.cpp:27-45: scale and zero point have x's rank, sizes 1 or x's.
namespace {
void check_linear_quantize_shapes(const Variables &inputs) {
  NBLA_CHECK((inputs[0]->ndim() == inputs[1]->ndim()) && (inputs[0]->ndim() == inputs[2]->ndim()), error_code::value,
             "Dimensions of inputs must be same (%d, %d, %d).", (int)inputs[0]->ndim(), (int)inputs[1]->ndim(),
             (int)inputs[2]->ndim());
  for (int i = 0; i < (int)inputs[0]->ndim(); ++i) {
    const auto s0 = inputs[0]->shape()[i], s1 = inputs[1]->shape()[i], s2 = inputs[2]->shape()[i];
    NBLA_CHECK(s1 == 1 || s1 == s0, error_code::value,
               "Size at %d-th dimension of inputs[1] (%d) should be 1 or match the size at %d-th dimension of "
               "inputs[0] (%d).",
               i, (int)s1, i, (int)s0);
    NBLA_CHECK(s2 == 1 || s2 == s0, error_code::value,
               "Size at %d-th dimension of inputs[2] (%d) should be 1 or match the size at %d-th dimension of "
               "inputs[0] (%d).",
               i, (int)s2, i, (int)s0);
  }
}
} // namespace

// quantize_linear.cpp:25-95
template <typename T> void QuantizeLinearHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  check_linear_quantize_shapes(inputs);
  NBLA_CHECK(this->round_mode_ == "HALF_AWAY_FROM_ZERO" || this->round_mode_ == "HALF_TO_EVEN", error_code::value,
             "round_mode must be HALF_AWAY_FROM_ZERO or HALF_TO_EVEN, not '%s'.", this->round_mode_.c_str());
  outputs[0]->reshape(inputs[0]->shape(), true);
  const dtypes dtype = static_cast<dtypes>(this->dtype_);
  if (dtype == dtypes::BYTE) {
    this->min_range_ = this->narrow_range_ ? -127 : -128;
    this->max_range_ = 127;
  } else if (dtype == dtypes::UBYTE) {
    this->min_range_ = this->narrow_range_ ? 1 : 0;
    this->max_range_ = 255;
  } else {
    NBLA_ERROR(error_code::value, "dtype must be BYTE (%d) or UBYTE (%d), not %d.", (int)dtypes::BYTE,
               (int)dtypes::UBYTE, this->dtype_);
  }
}

// dequantize_linear.cpp:25-53
template <typename T> void DequantizeLinearHip<T>::setup_impl(const Variables &inputs, const Variables &outputs) {
  check_linear_quantize_shapes(inputs);
  outputs[0]->reshape(inputs[0]->shape(), true);
}

// quantize_linear.cpp:97-117
template <typename T> void QuantizeLinearHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *scale = inputs[1]->get_data_pointer<T>(this->ctx_);
  T *zp = inputs[2]->cast_data_and_get_pointer<T>(this->ctx_, false); // rounded and saturated in place
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const vector<int64_t> xs = shape64(inputs[0]), ss = shape64(inputs[1]), zs = shape64(inputs[2]);
  NBLA_HIP_CALL(nbla_hip_quantize_linear_f32(x, scale, zp, y, xs.data(), ss.data(), zs.data(), (int)xs.size(),
                                             this->round_mode_ == "HALF_TO_EVEN", this->narrow_range_, this->dtype_,
                                             nullptr));
}

// quantize_linear.cpp:119-156
template <typename T>
void QuantizeLinearHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                         const vector<bool> &propagate_down, const vector<bool> &accum) {
  if (!(propagate_down[0] || propagate_down[1] || propagate_down[2]))
    return;
  if (propagate_down[0]) {
    hip_set_device(this->ctx_);
    const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
    const T *scale = inputs[1]->get_data_pointer<T>(this->ctx_);
    T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
    const vector<int64_t> xs = shape64(inputs[0]), ss = shape64(inputs[1]);
    NBLA_HIP_CALL(nbla_hip_quantize_linear_backward_f32(dy, scale, dx, xs.data(), ss.data(), (int)xs.size(), accum[0],
                                                        nullptr));
  }
  NBLA_CHECK(!propagate_down[1], error_code::not_implemented, "Backward w.r.t. the scale is not supported now.");
  NBLA_CHECK(!propagate_down[2], error_code::not_implemented, "Backward w.r.t. the zero point is not supported now.");
}

// dequantize_linear.cpp:55-67
template <typename T> void DequantizeLinearHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  const T *scale = inputs[1]->get_data_pointer<T>(this->ctx_);
  const T *zp = inputs[2]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  const vector<int64_t> xs = shape64(inputs[0]), ss = shape64(inputs[1]), zs = shape64(inputs[2]);
  NBLA_HIP_CALL(nbla_hip_dequantize_linear_f32(x, scale, zp, y, xs.data(), ss.data(), zs.data(), (int)xs.size(),
                                               nullptr));
}

// dequantize_linear.cpp:69-108
template <typename T>
void DequantizeLinearHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                           const vector<bool> &propagate_down, const vector<bool> &accum) {
  if (!(propagate_down[0] || propagate_down[1] || propagate_down[2]))
    return;
  if (propagate_down[0]) {
    hip_set_device(this->ctx_);
    const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
    const T *scale = inputs[1]->get_data_pointer<T>(this->ctx_);
    T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
    const vector<int64_t> xs = shape64(inputs[0]), ss = shape64(inputs[1]);
    NBLA_HIP_CALL(nbla_hip_dequantize_linear_backward_f32(dy, scale, dx, xs.data(), ss.data(), (int)xs.size(),
                                                          accum[0], nullptr));
  }
  NBLA_CHECK(!propagate_down[1], error_code::not_implemented, "Backward w.r.t. the scale is not supported now.");
  NBLA_CHECK(!propagate_down[2], error_code::not_implemented, "Backward w.r.t. the zero point is not supported now.");
}

// prune.cpp:39-70
template <typename T> void PruneHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  HipWorkspace ws(nbla_hip_prune_workspace_bytes(), this->ctx_);
  NBLA_HIP_CALL(nbla_hip_prune_f32(x, y, (size_t)inputs[0]->size(), this->rate_, ws.pointer(), ws.bytes(), nullptr));
}

// prune.cpp:72-90: the gradient passes through unchanged
template <typename T>
void PruneHip<T>::backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                                const vector<bool> &accum) {
  if (!propagate_down[0])
    return;
  hip_set_device(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  NBLA_HIP_CALL(nbla_hip_fixed_point_quantize_backward_f32(dy, dy, dx, (size_t)inputs[0]->size(), 1, 8, 1.0f, 0,
                                                           accum[0], nullptr));
}

// The recorder PythonFunctions' forward_impl (qnn.py:73-84, :178-188, :289-300, :411-420, :509-518): y.copy_from(x),
// then the statistics take this batch's extrema.
template <typename T> void RangeRecorderHip<T>::forward_impl(const Variables &inputs, const Variables &outputs) {
  hip_set_device(this->ctx_);
  const T *x = inputs[0]->get_data_pointer<T>(this->ctx_);
  T *y = outputs[0]->cast_data_and_get_pointer<T>(this->ctx_, true);
  T *m = nullptr, *M = nullptr;
  if (this->training_) {
    if (this->two_sided())
      m = inputs[1]->cast_data_and_get_pointer<T>(this->ctx_, false);
    Variable *stat = inputs[this->two_sided() ? 2 : 1];
    M = stat->cast_data_and_get_pointer<T>(this->ctx_, false);
  }
  HipWorkspace ws(nbla_hip_range_recorder_workspace_bytes(), this->ctx_);
  NBLA_HIP_CALL(nbla_hip_range_recorder_f32(x, y, (size_t)inputs[0]->size(), m, M, this->mode_, this->decay_,
                                            this->training_, ws.pointer(), ws.bytes(), nullptr));
}

// The gradient passes through unchanged.  (The reference's backward_impl, e.g. qnn.py:86-95, first copies the input
// gradient over the output gradient and so hands the input gradient back to itself; the recorders are identity
// functions and this is their gradient.)
template <typename T>
void RangeRecorderHip<T>::backward_impl(const Variables &inputs, const Variables &outputs,
                                        const vector<bool> &propagate_down, const vector<bool> &accum) {
  if (!propagate_down[0])
    return;
  hip_set_device(this->ctx_);
  const T *dy = outputs[0]->get_grad_pointer<T>(this->ctx_);
  T *dx = inputs[0]->cast_grad_and_get_pointer<T>(this->ctx_, !accum[0]);
  NBLA_HIP_CALL(nbla_hip_fixed_point_quantize_backward_f32(dy, dy, dx, (size_t)inputs[0]->size(), 1, 8, 1.0f, 0,
                                                           accum[0], nullptr));
}

// explicit instantiations for the "float" type config (function_types.yaml:483-509)
template class FixedPointQuantizeHip<float>;
template class Pow2QuantizeHip<float>;
template class MinMaxQuantizeHip<float>;
template class BinaryWeightAffineHip<float>;
template class BinaryConnectAffineHip<float>;
template class BinaryWeightConvolutionHip<float>;
template class BinaryConnectConvolutionHip<float>;
template class INQAffineHip<float, int>;
template class INQConvolutionHip<float, int>;
template class AffineHip<float>;
template class ReLUHip<float>;
template class Add2Hip<float>;
template class Sub2Hip<float>;
template class Pow2Hip<float>;
template class Mul2Hip<float>;
template class Div2Hip<float>;
template class ConcatenateHip<float>;
template class ConvolutionHip<float>;
template class QuantizeLinearHip<float>;
template class DequantizeLinearHip<float>;
template class PruneHip<float>;
template class SinkHip<float>;
template class RangeRecorderHip<float>;

} // namespace nbla
