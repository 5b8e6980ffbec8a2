// MinMaxQuantize (mirrors include/nbla/function/min_max_quantize.hpp:51-123).
#ifndef NBLA_FUNCTION_MIN_MAX_QUANTIZE_HPP_
#define NBLA_FUNCTION_MIN_MAX_QUANTIZE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(MinMaxQuantize, float, bool, bool, bool, float);

template <typename T> class MinMaxQuantize : public BaseFunction<float, bool, bool, bool, float> {
protected:
  const float decay_;
  const bool x_min_max_, ema_, ste_fine_grained_;
  const float eps_;
  VariablePtr scale_sptr_; // kept for backward, as in the reference

public:
  MinMaxQuantize(const Context &ctx, float decay, bool x_min_max, bool ema, bool ste_fine_grained, float eps)
      : BaseFunction(ctx, decay, x_min_max, ema, ste_fine_grained, eps), decay_(decay), x_min_max_(x_min_max),
        ema_(ema), ste_fine_grained_(ste_fine_grained), eps_(eps) {}
  virtual ~MinMaxQuantize() {}
  virtual shared_ptr<Function> copy() const {
    return create_MinMaxQuantize(ctx_, decay_, x_min_max_, ema_, ste_fine_grained_, eps_);
  }
  virtual int min_inputs() { return 5; }
  virtual int min_outputs() { return 1; }
  virtual vector<dtypes> in_types() {
    return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>(), get_dtype<T>(), get_dtype<T>()};
  }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual string name() { return "MinMaxQuantize"; }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }
  VariablePtr scale() { return scale_sptr_; }

protected:
  // min_max_quantize.cpp:45-127 (shape checks; the helper Functions the CPU class creates are not needed here)
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    auto x = inputs[0];
    auto qr_min = inputs[1], qr_max = inputs[2], ql_min = inputs[3], ql_max = inputs[4];
    NBLA_CHECK(ql_min->ndim() == ql_max->ndim() && ql_max->ndim() == qr_min->ndim() &&
                   qr_min->ndim() == qr_max->ndim(),
               error_code::value, "All input dimensions must be same.");
    NBLA_CHECK(ql_min->shape() == ql_max->shape() && ql_max->shape() == qr_min->shape() &&
                   qr_min->shape() == qr_max->shape(),
               error_code::value, "All shapes among ql_min, ql_max, qr_min, and qr_max must be same.");
    NBLA_CHECK(x->ndim() == ql_min->ndim(), error_code::value, "x and ql_min must have the same number of dimensions.");
    for (Size_t i = 0; i < ql_min->ndim(); i++) {
      NBLA_CHECK(ql_min->shape()[i] == 1 || x->shape()[i] == ql_min->shape()[i], error_code::value,
                 "x.shape and ql_min.shape must be same except for i-th dimension where ql_min.shape[i] == 1.");
    }
    outputs[0]->reshape(x->shape(), true);
    scale_sptr_ = make_shared<Variable>(ql_min->shape());
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("MinMaxQuantize"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("MinMaxQuantize backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return ste_fine_grained_ || !(x_min_max_ || ema_); }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return (i == 1 || i == 2) && x_min_max_; }
};

} // namespace nbla
#endif
