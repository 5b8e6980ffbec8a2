// FixedPointQuantize: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/fixed_point_quantize.hpp:39-89.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_FIXED_POINT_QUANTIZE_HPP_
#define NBLA_FUNCTION_FIXED_POINT_QUANTIZE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

#include <cmath>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(FixedPointQuantize, bool, int, float, bool);

// Inputs: x.
template <typename T> class FixedPointQuantize : public BaseFunction<bool, int, float, bool> {
protected:
  const bool sign_;
  const int n_;
  const float delta_;
  const bool ste_fine_grained_;
  float max_; // upper bound of the fixed-point range
  float min_; // lower bound

public:
  FixedPointQuantize(const Context &ctx, bool sign, int n, float delta, bool ste_fine_grained)
        : BaseFunction(ctx, sign, n, delta, ste_fine_grained), sign_(sign), n_(n), delta_(delta),
        ste_fine_grained_(ste_fine_grained) {}
  virtual ~FixedPointQuantize() {}
  virtual shared_ptr<Function> copy() const { return create_FixedPointQuantize(ctx_, sign_, n_, delta_,
      ste_fine_grained_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "FixedPointQuantize"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // fixed_point_quantize.cpp:29-43
    NBLA_CHECK(n_ > 0 && delta_ > 0., error_code::value, "Both bit width and delta should be positive.");
    outputs[0]->reshape(inputs[0]->shape(), true);
    const int n = sign_ ? n_ - 1 : n_;
    max_ = (float)((std::pow(2, n) - 1) * delta_);
    min_ = sign_ ? (T)(-max_) : (T)0;
    NBLA_CHECK(n > 0, error_code::value, "bit width should be positive when considering sign (1bit).");
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("FixedPointQuantize"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("FixedPointQuantize backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return ste_fine_grained_; }
};

} // namespace nbla
#endif
