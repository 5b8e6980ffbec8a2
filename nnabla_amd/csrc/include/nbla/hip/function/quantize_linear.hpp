// "hip:float" implementations of QuantizeLinear, DequantizeLinear and Prune.  The two linear quantizers replace the
// generic setup_impl (which also builds CPU helper functions); Prune reuses it.
#ifndef NBLA_HIP_FUNCTION_QUANTIZE_LINEAR_HPP_
#define NBLA_HIP_FUNCTION_QUANTIZE_LINEAR_HPP_

#include <nbla/function/dequantize_linear.hpp>
#include <nbla/function/prune.hpp>
#include <nbla/function/quantize_linear.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class QuantizeLinearHip : public QuantizeLinear<T> {
public:
  QuantizeLinearHip(const Context &ctx, const string &round_mode, bool narrow_range, int dtype)
      : QuantizeLinear<T>(ctx, round_mode, narrow_range, dtype) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class DequantizeLinearHip : public DequantizeLinear<T> {
public:
  DequantizeLinearHip(const Context &ctx)
      : DequantizeLinear<T>(ctx) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs);
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class PruneHip : public Prune<T> {
public:
  PruneHip(const Context &ctx, float rate)
      : Prune<T>(ctx, rate) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

} // namespace nbla
#endif
