// Shape inference of the affine- and convolution-shaped hip functions (checks and messages of the generic classes).
#include <nbla/hip/function/shapes.hpp>
#include <nbla/utils/axis_utils.hpp>

namespace nbla {

AffineShapes infer_affine_shapes(int base_axis, Variable *x, Variable *w, Variable *bias) {
  AffineShapes s;
  const Shape_t shape_data = x->shape();
  const Shape_t shape_weights = w->shape();
  NBLA_CHECK(shape_weights.size() >= 2, error_code::value, "Weights(inputs[1]) must be matrix or tensor.");
  refine_axis(base_axis, (int)x->ndim());
  s.base_axis = base_axis;
  NBLA_CHECK((size_t)base_axis < shape_data.size(), error_code::value,
             "Base_axis must be less than ndim of input data(inputs[0]). base_axis: %d >= ndim of input: %d.",
             base_axis, (int)shape_data.size());
  NBLA_CHECK(x->size(base_axis) == shape_weights[0], error_code::value,
             "Size of input data(inputs[0]) and weights(inputs[1]) mismatch. size of input: %ld != size of weights: %ld.",
             (long)x->size(base_axis), (long)shape_weights[0]);
  s.i_col = x->size(base_axis);
  s.i_row = s.i_col ? x->size() / s.i_col : 0;
  s.w_row = shape_weights[0];
  s.w_col = s.w_row ? w->size() / s.w_row : 0;
  for (int i = 0; i < base_axis; ++i)
    s.out_shape.push_back(shape_data[i]);
  for (size_t i = 1; i < shape_weights.size(); ++i)
    s.out_shape.push_back(shape_weights[i]);
  if (bias) {
    const Shape_t shape_bias = bias->shape();
    NBLA_CHECK(shape_bias.size() == shape_weights.size() - 1, error_code::value,
               "Length of bias(inputs[2]) and weights(inputs[1]) mismatch. bias length: %d != weights length-1: %d.",
               (int)shape_bias.size(), (int)shape_weights.size() - 1);
    for (size_t i = 0; i < shape_bias.size(); ++i)
      NBLA_CHECK(shape_bias[i] == shape_weights[i + 1], error_code::value,
                 "Shape of bias(inputs[2]) and weights(inputs[1]) mismatch.");
  }
  return s;
}

ConvShapes infer_conv_shapes(int base_axis, const vector<int> &pad, const vector<int> &stride,
                             const vector<int> &dilation, int group, Variable *x, Variable *w, Variable *bias) {
  ConvShapes s;
  const Shape_t shape_data = x->shape();
  const Shape_t shape_weights = w->shape();
  refine_axis(base_axis, (int)x->ndim());
  s.base_axis = base_axis;
  NBLA_CHECK((size_t)base_axis < shape_data.size() - 1, error_code::unclassified,
             "base_axis must be less than ndim - 1 of inputs[0]. base_axis: %d >= ndim of inputs[0] - 1: %d.",
             base_axis, (int)shape_data.size() - 1);
  const size_t spatial_dims = shape_data.size() - base_axis - 1;
  NBLA_CHECK(shape_weights.size() == 2 + spatial_dims, error_code::value, "Weights must be a tensor more than 3D.");
  s.spatial_dims = (int)spatial_dims;
  s.group = group;
  s.channels_i = shape_data[base_axis];
  s.channels_o = shape_weights[0];
  s.channels_g = shape_weights[1];
  NBLA_CHECK(group > 0 && s.channels_i % group == 0, error_code::value,
             "Number of input channel needs to be divisible by group. Input channel: %ld, group: %d.",
             (long)s.channels_i, group);
  NBLA_CHECK(s.channels_o % group == 0, error_code::value,
             "Number of output channel needs to be divisible by group. Output channel: %ld, group: %d.",
             (long)s.channels_o, group);
  NBLA_CHECK(s.channels_i / group == s.channels_g, error_code::value,
             "Number of grouped channel mismatch. Input: %ld != Weights[1]: %ld.", (long)(s.channels_i / group),
             (long)s.channels_g);
  NBLA_CHECK(pad.size() == spatial_dims, error_code::value, "pad size mismatch. pad size: %d != spatial dims: %d.",
             (int)pad.size(), (int)spatial_dims);
  NBLA_CHECK(stride.size() == spatial_dims, error_code::value,
             "stride size mismatch. stride size: %d != spatial dims: %d.", (int)stride.size(), (int)spatial_dims);
  NBLA_CHECK(dilation.size() == spatial_dims, error_code::value,
             "dilation size mismatch. dilation size: %d != spatial dims: %d.", (int)dilation.size(),
             (int)spatial_dims);
  s.inner_size_k = s.channels_g;
  s.outer = 1;
  s.out_shape = Shape_t(shape_data.size());
  for (int i = 0; i < base_axis; ++i) {
    s.out_shape[i] = shape_data[i];
    s.outer *= shape_data[i];
  }
  s.out_shape[base_axis] = s.channels_o;
  for (size_t i = 0; i < spatial_dims; ++i) {
    const int64_t kernel = shape_weights[2 + i];
    const int64_t in = shape_data[base_axis + 1 + i];
    const int64_t k = dilation[i] * (kernel - 1) + 1;
    const int64_t o = (in + 2 * pad[i] - k) / stride[i] + 1;
    NBLA_CHECK(o > 0 && in + 2 * pad[i] - k >= 0, error_code::value,
               "Invalid configuration of convolution at %d-th spatial dimension.  {input:%ld, kernel:%ld, pad:%d, "
               "stride:%d, dilation:%d}.",
               (int)i, (long)in, (long)kernel, pad[i], stride[i], dilation[i]);
    s.kernel.push_back(kernel);
    s.pad.push_back(pad[i]);
    s.stride.push_back(stride[i]);
    s.dilation.push_back(dilation[i]);
    s.spatial_i.push_back(in);
    s.spatial_o.push_back(o);
    s.inner_size_k *= kernel;
    s.out_shape[base_axis + 1 + i] = o;
  }
  if (bias) {
    NBLA_CHECK(bias->shape().size() == 1, error_code::value, "Bias(inputs[2]) must be a 1d tensor.");
    NBLA_CHECK(bias->shape()[0] == s.channels_o, error_code::value,
               "Shape of bias(inputs[2]) and weights(inputs[1]) mismatch. bias shape[0]: %ld != weights shape[0]: %ld.",
               (long)bias->shape()[0], (long)s.channels_o);
  }
  return s;
}

} // namespace nbla
