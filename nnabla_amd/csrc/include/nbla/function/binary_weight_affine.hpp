// BinaryWeightAffine: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/binary_weight_affine.hpp:72-123.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_BINARY_WEIGHT_AFFINE_HPP_
#define NBLA_FUNCTION_BINARY_WEIGHT_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(BinaryWeightAffine, int, float);

// Inputs: x, weight, binary_weight (written), alpha (written), [bias].
template <typename T> class BinaryWeightAffine : public BaseFunction<int> {
protected:
  int base_axis_;
  float quantize_zero_to_;
  Size_t w_row_, w_col_;

public:
  BinaryWeightAffine(const Context &ctx, int base_axis, float quantize_zero_to)
        : BaseFunction(ctx, base_axis), base_axis_(base_axis), quantize_zero_to_(quantize_zero_to) {}
  virtual ~BinaryWeightAffine() {}
  virtual shared_ptr<Function> copy() const { return create_BinaryWeightAffine(ctx_, base_axis_, quantize_zero_to_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>(),
      get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 4; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "BinaryWeightAffine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("BinaryWeightAffine"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("BinaryWeightAffine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("BinaryWeightAffine backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return i == 1 && j == 0; }
};

} // namespace nbla
#endif
