// Pow2: the class a "hip:float" implementation derives from.  Constructor, argument types and member names are
// those the reference's include/nbla/function/pow2.hpp:44 declares through NBLA_DEFINE_TRANSFORM_BINARY_INPLACE.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_POW2_HPP_
#define NBLA_FUNCTION_POW2_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function/utils/base_transform_binary.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Pow2, bool);

// Inputs: x0, x1.  y = x0 ^ x1, element by element.
template <typename T> class Pow2 : public BaseFunction<bool> {
public:
  Pow2(const Context &ctx, bool inplace) : BaseFunction(ctx, inplace) {}
  virtual ~Pow2() {}
  virtual shared_ptr<Function> copy() const { return create_Pow2(ctx_, false /* inplace is obsolete */); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Pow2"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // utils/base_transform_binary.hpp:58-86 (the in-place form is obsolete: copy() above never asks for it)
    transform_binary_setup(inputs, outputs, false, this->name());
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Pow2"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Pow2 backward");
  }
  // the gradient with respect to either input reads both inputs (pow2.hpp:44-47)
  virtual bool grad_depends_input_data_impl(int i, int j) const { return true; }
};

} // namespace nbla
#endif
