// Shape inference of the affine- and convolution-shaped "hip:float" functions.  The generic classes of nnabla infer
// these inside setup_impl bodies that also build chains of CPU helper functions; the hip classes replace those
// bodies, so they carry the inferred geometry themselves, in the form the kernel library takes it.
#ifndef NBLA_HIP_FUNCTION_SHAPES_HPP_
#define NBLA_HIP_FUNCTION_SHAPES_HPP_

#include <nbla/function.hpp>

namespace nbla {

// Affine<T>::setup_impl (src/nbla/function/generic/affine.cpp:29-78): x [.., i_col] viewed [i_row, i_col],
// W [w_row, ...] viewed [w_row, w_col]; output shape x.shape[:base_axis] + W.shape[1:].  Same checks and messages.
struct AffineShapes {
  int base_axis;
  Size_t i_row, i_col, w_row, w_col;
  Shape_t out_shape;
};
NBLA_API AffineShapes infer_affine_shapes(int base_axis, Variable *x, Variable *w, Variable *bias);

// Convolution<T>::setup_impl (src/nbla/function/generic/convolution.cpp:41-160), channel-first.
struct ConvShapes {
  int base_axis, spatial_dims;
  Size_t outer, channels_i, channels_o, channels_g, group, inner_size_k;
  vector<int64_t> kernel, pad, stride, dilation, spatial_i, spatial_o;
  Shape_t out_shape;
};
NBLA_API ConvShapes infer_conv_shapes(int base_axis, const vector<int> &pad, const vector<int> &stride,
                                      const vector<int> &dilation, int group, Variable *x, Variable *w, Variable *bias);

} // namespace nbla
#endif
