// Affine: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/affine.hpp:50-107.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_AFFINE_HPP_
#define NBLA_FUNCTION_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Affine, int);

// Inputs: x, weight, [bias].
template <typename T> class Affine : public BaseFunction<int> {
protected:
  int base_axis_;
  Size_t i_row_, i_col_, w_row_, w_col_, o_row_, o_col_;

public:
  Affine(const Context &ctx, int base_axis) : BaseFunction(ctx, base_axis), base_axis_(base_axis) {}
  virtual ~Affine() {}
  virtual shared_ptr<Function> copy() const { return create_Affine(ctx_, base_axis_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Affine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Affine"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Affine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Affine backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return (i == 0 && j == 1) || (i == 1 && j == 0); }
};

} // namespace nbla
#endif
