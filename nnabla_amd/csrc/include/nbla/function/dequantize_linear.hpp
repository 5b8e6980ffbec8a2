// DequantizeLinear: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/dequantize_linear.hpp:38-86.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_DEQUANTIZE_LINEAR_HPP_
#define NBLA_FUNCTION_DEQUANTIZE_LINEAR_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(DequantizeLinear);

// Inputs: x, scale, zero_point.
template <typename T> class DequantizeLinear : public BaseFunction<> {
public:
  DequantizeLinear(const Context &ctx) : BaseFunction(ctx) {}
  virtual ~DequantizeLinear() {}
  virtual shared_ptr<Function> copy() const { return create_DequantizeLinear(ctx_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 3; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "DequantizeLinear"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("DequantizeLinear"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("DequantizeLinear"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("DequantizeLinear backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return i == 0 && j == 1; }
};

} // namespace nbla
#endif
