// Add2: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/add2.hpp:27-80.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_ADD2_HPP_
#define NBLA_FUNCTION_ADD2_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function/utils/base_transform_binary.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Add2, bool);

// Inputs: x0, x1.
template <typename T> class Add2 : public BaseFunction<bool> {
public:
  Add2(const Context &ctx, bool inplace) : BaseFunction(ctx, inplace) {}
  virtual ~Add2() {}
  virtual shared_ptr<Function> copy() const { return create_Add2(ctx_, false /* inplace is obsolete */); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Add2"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // add2.cpp:28-37: inputs of one shape, or the broadcasting form (BcAdd2: utils/base_transform_binary.hpp:58-86)
    if (inputs[0]->shape() == inputs[1]->shape()) {
      outputs[0]->reshape(inputs[0]->shape(), true);
      return;
    }
    transform_binary_setup(inputs, outputs, false, this->name());
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Add2"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Add2 backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

} // namespace nbla
#endif
