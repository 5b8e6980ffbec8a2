// Affine and ReLU: the two plain functions the quantized graphs of this build need beside the quantization family
// (mirrors include/nbla/function/affine.hpp and relu.hpp).
#ifndef NBLA_FUNCTION_AFFINE_HPP_
#define NBLA_FUNCTION_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Affine, int);
NBLA_REGISTER_FUNCTION_HEADER(ReLU, bool);

// Inputs: x, weight, [bias].
template <typename T> class Affine : public BaseFunction<int> {
protected:
  int base_axis_;
  AffineShapes shapes_;

public:
  Affine(const Context &ctx, int base_axis) : BaseFunction(ctx, base_axis), base_axis_(base_axis) {}
  virtual ~Affine() {}
  virtual shared_ptr<Function> copy() const { return create_Affine(ctx_, base_axis_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Affine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    shapes_ = infer_affine_shapes(base_axis_, inputs[0], inputs[1], inputs.size() == 3 ? inputs[2] : nullptr);
    base_axis_ = shapes_.base_axis;
    outputs[0]->reshape(shapes_.out_shape, true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Affine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Affine backward");
  }
};

template <typename T> class ReLU : public BaseFunction<bool> {
protected:
  bool inplace_;

public:
  ReLU(const Context &ctx, bool inplace) : BaseFunction(ctx, inplace), inplace_(inplace) {}
  virtual ~ReLU() {}
  virtual shared_ptr<Function> copy() const { return create_ReLU(ctx_, inplace_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "ReLU"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_input_data(int i, int j) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("ReLU"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("ReLU backward");
  }
};

} // namespace nbla
#endif
