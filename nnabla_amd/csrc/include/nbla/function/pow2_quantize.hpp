// Pow2Quantize: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/pow2_quantize.hpp:45-101.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_POW2_QUANTIZE_HPP_
#define NBLA_FUNCTION_POW2_QUANTIZE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

#include <cmath>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Pow2Quantize, bool, bool, int, int, bool);

// Inputs: x.
template <typename T> class Pow2Quantize : public BaseFunction<bool, bool, int, int, bool> {
protected:
  const bool sign_;
  const bool with_zero_;
  const int n_;
  const int m_;
  const bool ste_fine_grained_;
  float p_max_; // upper bound in the positive region
  float p_min_; // lower bound in the positive region
  float pruning_threshold_;

public:
  Pow2Quantize(const Context &ctx, bool sign, bool with_zero, int n, int m, bool ste_fine_grained)
        : BaseFunction(ctx, sign, with_zero, n, m, ste_fine_grained), sign_(sign), with_zero_(with_zero), n_(n),
        m_(m), ste_fine_grained_(ste_fine_grained) {}
  virtual ~Pow2Quantize() {}
  virtual shared_ptr<Function> copy() const { return create_Pow2Quantize(ctx_, sign_, with_zero_, n_, m_,
      ste_fine_grained_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Pow2Quantize"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // pow2_quantize.cpp:29-45
    NBLA_CHECK(n_ > 0, error_code::value, "bit width should be positive.");
    outputs[0]->reshape(inputs[0]->shape(), true);
    int n = sign_ ? n_ - 1 : n_;
    n = with_zero_ ? n - 1 : n;
    int ref_p_max = m_;
    int ref_p_min = m_ - ((1 << n) - 1);
    p_max_ = std::pow(2., ref_p_max);
    p_min_ = std::pow(2., ref_p_min);
    pruning_threshold_ = p_min_ * std::pow(2., -0.5);
    NBLA_CHECK(n > 0, error_code::value, "bit width should be positive when considering zero and sign (1bit each).");
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Pow2Quantize"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Pow2Quantize backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return ste_fine_grained_; }
};

} // namespace nbla
#endif
