// "hip:float" implementations of INQAffine / INQConvolution and of the plain functions (Affine, Convolution, ReLU)
// that the quantized graphs need.  setup_impl replaces the generic one wherever that one would build CPU helper
// functions or where the kernel library wants the geometry in its own form.
#ifndef NBLA_HIP_FUNCTION_INQ_HPP_
#define NBLA_HIP_FUNCTION_INQ_HPP_

#include <nbla/function/affine.hpp>
#include <nbla/function/convolution.hpp>
#include <nbla/function/inq_affine.hpp>
#include <nbla/function/inq_convolution.hpp>
#include <nbla/function/relu.hpp>
#include <nbla/hip/function/shapes.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T, typename T1> class INQAffineHip : public INQAffine<T, T1> {
protected:
  AffineShapes shapes_; // filled by setup_impl

public:
  INQAffineHip(const Context &ctx, int base_axis, int num_bits, const vector<int> &inq_iterations,
               const string &selection_algorithm, int seed)
      : INQAffine<T, T1>(ctx, base_axis, num_bits, inq_iterations, selection_algorithm, seed) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs);
  void run(const Variables &inputs, const Variables &outputs, int step);
};

template <typename T, typename T1> class INQConvolutionHip : public INQConvolution<T, T1> {
protected:
  ConvShapes shapes_; // filled by setup_impl

public:
  INQConvolutionHip(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
                    const vector<int> &dilation, int group, int num_bits, const vector<int> &inq_iterations,
                    const string &selection_algorithm, int seed)
      : INQConvolution<T, T1>(ctx, base_axis, pad, stride, dilation, group, num_bits, inq_iterations,
                              selection_algorithm, seed) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs);
  void run(const Variables &inputs, const Variables &outputs, int step);
};

template <typename T> class AffineHip : public Affine<T> {
protected:
  AffineShapes shapes_; // filled by setup_impl

public:
  AffineHip(const Context &ctx, int base_axis)
      : Affine<T>(ctx, base_axis) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class ConvolutionHip : public Convolution<T> {
protected:
  ConvShapes shapes_; // filled by setup_impl

public:
  ConvolutionHip(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
                 const vector<int> &dilation, int group, bool channel_last)
      : Convolution<T>(ctx, base_axis, pad, stride, dilation, group, channel_last) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class ReLUHip : public ReLU<T> {
public:
  ReLUHip(const Context &ctx, bool inplace)
      : ReLU<T>(ctx, inplace) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

} // namespace nbla
#endif
