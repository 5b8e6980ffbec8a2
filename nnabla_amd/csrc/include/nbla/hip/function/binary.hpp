// "hip:float" implementations of the binary-weight functions.  Their setup_impl replaces the generic one (which, in
// nnabla, also builds the chain of CPU helper functions): same argument checks, and the geometry kept in the form
// the kernel library takes it.
#ifndef NBLA_HIP_FUNCTION_BINARY_HPP_
#define NBLA_HIP_FUNCTION_BINARY_HPP_

#include <nbla/function/binary_connect_affine.hpp>
#include <nbla/function/binary_connect_convolution.hpp>
#include <nbla/function/binary_weight_affine.hpp>
#include <nbla/function/binary_weight_convolution.hpp>
#include <nbla/hip/function/shapes.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class BinaryWeightAffineHip : public BinaryWeightAffine<T> {
protected:
  AffineShapes shapes_; // filled by setup_impl

public:
  BinaryWeightAffineHip(const Context &ctx, int base_axis, float quantize_zero_to)
      : BinaryWeightAffine<T>(ctx, base_axis, quantize_zero_to) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 2 || i == 3; }
};

template <typename T> class BinaryConnectAffineHip : public BinaryConnectAffine<T> {
protected:
  AffineShapes shapes_; // filled by setup_impl

public:
  BinaryConnectAffineHip(const Context &ctx, int base_axis, float quantize_zero_to)
      : BinaryConnectAffine<T>(ctx, base_axis, quantize_zero_to) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 2; }
};

template <typename T> class BinaryWeightConvolutionHip : public BinaryWeightConvolution<T> {
protected:
  ConvShapes shapes_; // filled by setup_impl

public:
  BinaryWeightConvolutionHip(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
                             const vector<int> &dilation, int group, float quantize_zero_to)
      : BinaryWeightConvolution<T>(ctx, base_axis, pad, stride, dilation, group, quantize_zero_to) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 2 || i == 3; }
};

template <typename T> class BinaryConnectConvolutionHip : public BinaryConnectConvolution<T> {
protected:
  ConvShapes shapes_; // filled by setup_impl

public:
  BinaryConnectConvolutionHip(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
                              const vector<int> &dilation, int group, float quantize_zero_to)
      : BinaryConnectConvolution<T>(ctx, base_axis, pad, stride, dilation, group, quantize_zero_to) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 2; }
};

} // namespace nbla
#endif
