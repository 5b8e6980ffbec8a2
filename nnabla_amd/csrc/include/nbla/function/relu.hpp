// ReLU: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/relu.hpp:40-81.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_RELU_HPP_
#define NBLA_FUNCTION_RELU_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(ReLU, bool);

// Inputs: x.
template <typename T> class ReLU : public BaseFunction<bool> {
public:
  ReLU(const Context &ctx, bool inplace) : BaseFunction(ctx, inplace) {}
  virtual ~ReLU() {}
  virtual shared_ptr<Function> copy() const { return create_ReLU(ctx_, false /* inplace is obsolete */); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "ReLU"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return true; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // relu.cpp:30-33
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("ReLU"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("ReLU backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

} // namespace nbla
#endif
