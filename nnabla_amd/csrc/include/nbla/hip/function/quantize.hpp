// "hip:float" implementations of the elementwise quantizers.  FixedPointQuantize and Pow2Quantize reuse the generic
// setup_impl (argument checks and the derived bounds); MinMaxQuantize replaces it, because the generic one also builds
// the chain of CPU helper functions that its forward pass runs.
#ifndef NBLA_HIP_FUNCTION_QUANTIZE_HPP_
#define NBLA_HIP_FUNCTION_QUANTIZE_HPP_

#include <nbla/function/fixed_point_quantize.hpp>
#include <nbla/function/min_max_quantize.hpp>
#include <nbla/function/pow2_quantize.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class FixedPointQuantizeHip : public FixedPointQuantize<T> {
public:
  FixedPointQuantizeHip(const Context &ctx, bool sign, int n, float delta, bool ste_fine_grained)
      : FixedPointQuantize<T>(ctx, sign, n, delta, ste_fine_grained) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class Pow2QuantizeHip : public Pow2Quantize<T> {
public:
  Pow2QuantizeHip(const Context &ctx, bool sign, bool with_zero, int n, int m, bool ste_fine_grained)
      : Pow2Quantize<T>(ctx, sign, with_zero, n, m, ste_fine_grained) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class MinMaxQuantizeHip : public MinMaxQuantize<T> {
public:
  MinMaxQuantizeHip(const Context &ctx, float decay, bool x_min_max, bool ema, bool ste_fine_grained, float eps)
      : MinMaxQuantize<T>(ctx, decay, x_min_max, ema, ste_fine_grained, eps) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

} // namespace nbla
#endif
