// MinMaxQuantize: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/min_max_quantize.hpp:51-123.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_MIN_MAX_QUANTIZE_HPP_
#define NBLA_FUNCTION_MIN_MAX_QUANTIZE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(MinMaxQuantize, float, bool, bool, bool, float);

// Inputs: x, qr_min (state, rewritten), qr_max (state, rewritten), ql_min, ql_max.
template <typename T> class MinMaxQuantize : public BaseFunction<float, bool, bool, bool, float> {
protected:
  float decay_;
  bool x_min_max_;
  bool ema_;
  bool ste_fine_grained_;
  float eps_;
  VariablePtr scale_sptr_; // the scale of the last forward pass, read by the backward pass

public:
  MinMaxQuantize(const Context &ctx, float decay, bool x_min_max, bool ema, bool ste_fine_grained, float eps)
        : BaseFunction(ctx, decay, x_min_max, ema, ste_fine_grained, eps), decay_(decay), x_min_max_(x_min_max),
        ema_(ema), ste_fine_grained_(ste_fine_grained), eps_(eps) {}
  virtual ~MinMaxQuantize() {}
  virtual shared_ptr<Function> copy() const { return create_MinMaxQuantize(ctx_, decay_, x_min_max_, ema_,
      ste_fine_grained_, eps_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>(),
      get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 5; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "MinMaxQuantize"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("MinMaxQuantize"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("MinMaxQuantize"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("MinMaxQuantize backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return ste_fine_grained_ || !(x_min_max_ || ema_); }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return (i == 1 || i == 2) && x_min_max_; }
};

} // namespace nbla
#endif
