// QuantizeLinear, DequantizeLinear and Prune (mirror include/nbla/function/quantize_linear.hpp:43-100,
// dequantize_linear.hpp and prune.hpp): argument checks and shape inference; the arithmetic lives in the
// extension classes.
#ifndef NBLA_FUNCTION_QUANTIZE_LINEAR_HPP_
#define NBLA_FUNCTION_QUANTIZE_LINEAR_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(QuantizeLinear, const string &, bool, int);
NBLA_REGISTER_FUNCTION_HEADER(DequantizeLinear);
NBLA_REGISTER_FUNCTION_HEADER(Prune, float);

// quantize_linear.cpp:28-46 and dequantize_linear.cpp:27-45: scale and zero point have x's rank, sizes 1 or x's.
inline void check_linear_quantize_shapes(const Variables &inputs) {
  NBLA_CHECK((inputs[0]->ndim() == inputs[1]->ndim()) && (inputs[0]->ndim() == inputs[2]->ndim()), error_code::value,
             "Dimensions of inputs must be same (%d, %d, %d).", (int)inputs[0]->ndim(), (int)inputs[1]->ndim(),
             (int)inputs[2]->ndim());
  for (int i = 0; i < (int)inputs[0]->ndim(); ++i) {
    const auto s0 = inputs[0]->shape()[i], s1 = inputs[1]->shape()[i], s2 = inputs[2]->shape()[i];
    NBLA_CHECK(s1 == 1 || s1 == s0, error_code::value,
               "Size at %d-th dimension of inputs[1] (%d) should be 1 or match the size at %d-th dimension of "
               "inputs[0] (%d).",
               i, (int)s1, i, (int)s0);
    NBLA_CHECK(s2 == 1 || s2 == s0, error_code::value,
               "Size at %d-th dimension of inputs[2] (%d) should be 1 or match the size at %d-th dimension of "
               "inputs[0] (%d).",
               i, (int)s2, i, (int)s0);
  }
}

// Inputs: x, scale, zero_point (rounded and saturated in place by the forward pass).
template <typename T> class QuantizeLinear : public BaseFunction<const string &, bool, int> {
protected:
  string round_mode_;
  bool narrow_range_;
  int dtype_;
  int min_range_, max_range_;

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
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    check_linear_quantize_shapes(inputs);
    NBLA_CHECK(round_mode_ == "HALF_AWAY_FROM_ZERO" || round_mode_ == "HALF_TO_EVEN", error_code::value,
               "round_mode must be HALF_AWAY_FROM_ZERO or HALF_TO_EVEN, not '%s'.", round_mode_.c_str());
    outputs[0]->reshape(inputs[0]->shape(), true);
    const dtypes dtype = static_cast<dtypes>(dtype_);
    if (dtype == dtypes::BYTE) {
      min_range_ = narrow_range_ ? -127 : -128;
      max_range_ = 127;
    } else if (dtype == dtypes::UBYTE) {
      min_range_ = narrow_range_ ? 1 : 0;
      max_range_ = 255;
    } else {
      NBLA_ERROR(error_code::value, "dtype must be BYTE (%d) or UBYTE (%d), not %d.", (int)dtypes::BYTE,
                 (int)dtypes::UBYTE, dtype_);
    }
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("QuantizeLinear"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("QuantizeLinear backward");
  }
};

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
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    check_linear_quantize_shapes(inputs);
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("DequantizeLinear"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("DequantizeLinear backward");
  }
};

template <typename T> class Prune : public BaseFunction<float> {
protected:
  float rate_;
  int thresh_idx_;

public:
  Prune(const Context &ctx, float rate) : BaseFunction(ctx, rate), rate_(rate), thresh_idx_(0) {}
  virtual ~Prune() {}
  virtual shared_ptr<Function> copy() const { return create_Prune(ctx_, rate_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Prune"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }
  virtual bool grad_depends_input_data(int i, int j) const { return false; }

protected:
  // prune.cpp:27-37
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(rate_ >= 0 && rate_ <= 1, error_code::value, "Rate %f must be in [0, 1].", rate_);
    const int x_size = (int)inputs[0]->size();
    thresh_idx_ = (int)((x_size - 1) * this->rate_);
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Prune"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Prune backward");
  }
};

} // namespace nbla
#endif
