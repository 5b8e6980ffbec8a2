// Pow2Quantize (mirrors include/nbla/function/pow2_quantize.hpp:45-101).
#ifndef NBLA_FUNCTION_POW2_QUANTIZE_HPP_
#define NBLA_FUNCTION_POW2_QUANTIZE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

#include <cmath>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Pow2Quantize, bool, bool, int, int, bool);

template <typename T> class Pow2Quantize : public BaseFunction<bool, bool, int, int, bool> {
protected:
  const bool sign_, with_zero_;
  const int n_, m_;
  const bool ste_fine_grained_;
  float p_max_, p_min_, pruning_threshold_;

public:
  Pow2Quantize(const Context &ctx, bool sign, bool with_zero, int n, int m, bool ste_fine_grained)
      : BaseFunction(ctx, sign, with_zero, n, m, ste_fine_grained), sign_(sign), with_zero_(with_zero), n_(n), m_(m),
        ste_fine_grained_(ste_fine_grained) {}
  virtual ~Pow2Quantize() {}
  virtual shared_ptr<Function> copy() const {
    return create_Pow2Quantize(ctx_, sign_, with_zero_, n_, m_, ste_fine_grained_);
  }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Pow2Quantize"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  // pow2_quantize.cpp:29-45
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(n_ > 0, error_code::value, "bit width should be positive.");
    outputs[0]->reshape(inputs[0]->shape(), true);
    int n = sign_ ? n_ - 1 : n_;
    n = with_zero_ ? n - 1 : n;
    NBLA_CHECK(n > 0, error_code::value,
               "bit width should be positive when considering zero (1bit) and sign (1bit).");
    p_max_ = (float)std::pow(2., m_);
    p_min_ = (float)std::pow(2., m_ - ((1 << n) - 1));
    pruning_threshold_ = (float)(p_min_ * std::pow(2., -0.5));
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Pow2Quantize"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Pow2Quantize backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return ste_fine_grained_; }
};

} // namespace nbla
#endif
