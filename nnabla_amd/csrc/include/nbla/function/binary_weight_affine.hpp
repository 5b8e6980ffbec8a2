// BinaryWeightAffine (mirrors include/nbla/function/binary_weight_affine.hpp:72-123).
#ifndef NBLA_FUNCTION_BINARY_WEIGHT_AFFINE_HPP_
#define NBLA_FUNCTION_BINARY_WEIGHT_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(BinaryWeightAffine, int, float);

// Inputs: x, weight, binary_weight (written), alpha (written), [bias].
template <typename T> class BinaryWeightAffine : public BaseFunction<int, float> {
protected:
  int base_axis_;
  float quantize_zero_to_;
  AffineShapes shapes_;

public:
  BinaryWeightAffine(const Context &ctx, int base_axis, float quantize_zero_to)
      : BaseFunction(ctx, base_axis, quantize_zero_to), base_axis_(base_axis), quantize_zero_to_(quantize_zero_to) {}
  virtual ~BinaryWeightAffine() {}
  virtual shared_ptr<Function> copy() const { return create_BinaryWeightAffine(ctx_, base_axis_, quantize_zero_to_); }
  virtual vector<dtypes> in_types() {
    return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>(), get_dtype<T>(), get_dtype<T>()};
  }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 4; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "BinaryWeightAffine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  // binary_weight_affine.cpp:32-72
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    shapes_ = infer_affine_shapes(base_axis_, inputs[0], inputs[1], inputs.size() == 5 ? inputs[4] : nullptr);
    base_axis_ = shapes_.base_axis;
    NBLA_CHECK(inputs[1]->shape() == inputs[2]->shape(), error_code::value,
               "Binary and float weights must have same size.");
    NBLA_CHECK(inputs[3]->size() == shapes_.w_col, error_code::value, "Size of alpha must be equal to output size.");
    outputs[0]->reshape(shapes_.out_shape, true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("BinaryWeightAffine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("BinaryWeightAffine backward");
  }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 2 || i == 3; }
};

} // namespace nbla
#endif
