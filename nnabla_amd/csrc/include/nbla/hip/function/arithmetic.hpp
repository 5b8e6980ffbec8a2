// "hip:float" implementations of Add2 and Concatenate (the functions whose inputs share one quantization range in
// quantization-aware training) and of Sub2, Mul2, Div2, Pow2 (whose two inputs are both activations to it); all reuse
// the generic setup_impl, broadcasting included.
#ifndef NBLA_HIP_FUNCTION_ARITHMETIC_HPP_
#define NBLA_HIP_FUNCTION_ARITHMETIC_HPP_

#include <nbla/function/add2.hpp>
#include <nbla/function/concatenate.hpp>
#include <nbla/function/div2.hpp>
#include <nbla/function/mul2.hpp>
#include <nbla/function/pow2.hpp>
#include <nbla/function/sub2.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

template <typename T> class Add2Hip : public Add2<T> {
public:
  Add2Hip(const Context &ctx, bool inplace) : Add2<T>(ctx, inplace) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

template <typename T> class ConcatenateHip : public Concatenate<T> {
public:
  ConcatenateHip(const Context &ctx, int axis) : Concatenate<T>(ctx, axis) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

#define NBLA_HIP_DECLARE_BINARY2(NAME)                                                                                 \
  template <typename T> class NAME##Hip : public NAME<T> {                                                             \
  public:                                                                                                              \
    NAME##Hip(const Context &ctx, bool inplace) : NAME<T>(ctx, inplace) {}                                            \
    virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }          \
                                                                                                                       \
  protected:                                                                                                           \
    virtual void forward_impl(const Variables &inputs, const Variables &outputs);                                     \
    virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down, \
                               const vector<bool> &accum);                                                            \
  }
NBLA_HIP_DECLARE_BINARY2(Sub2);
NBLA_HIP_DECLARE_BINARY2(Mul2);
NBLA_HIP_DECLARE_BINARY2(Div2);
NBLA_HIP_DECLARE_BINARY2(Pow2);
#undef NBLA_HIP_DECLARE_BINARY2

} // namespace nbla
#endif
