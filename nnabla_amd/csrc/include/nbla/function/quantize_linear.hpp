// QuantizeLinear: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/quantize_linear.hpp:43-100.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_QUANTIZE_LINEAR_HPP_
#define NBLA_FUNCTION_QUANTIZE_LINEAR_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(QuantizeLinear, const string &, bool, int);

// Inputs: x, scale, zero_point (rounded and saturated in place by the forward pass).
template <typename T> class QuantizeLinear : public BaseFunction<const string &, bool, int> {
protected:
  string round_mode_;
  bool narrow_range_;
  int dtype_;

  int min_range_;
  int max_range_;

public:
  QuantizeLinear(const Context &ctx, const string &round_mode, bool narrow_range, int dtype)
        : BaseFunction(ctx, round_mode, narrow_range, dtype), round_mode_(round_mode), narrow_range_(narrow_range),
        dtype_(dtype), min_range_(0), max_range_(0) {}
  virtual ~QuantizeLinear() {}
  virtual shared_ptr<Function> copy() const { return create_QuantizeLinear(ctx_, round_mode_, narrow_range_, dtype_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 3; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "QuantizeLinear"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("QuantizeLinear"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("QuantizeLinear"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("QuantizeLinear backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return i == 0 && j == 1; }
};

} // namespace nbla
#endif
