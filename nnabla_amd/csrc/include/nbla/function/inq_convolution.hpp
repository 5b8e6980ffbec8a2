// INQConvolution (mirrors include/nbla/function/inq_convolution.hpp).
#ifndef NBLA_FUNCTION_INQ_CONVOLUTION_HPP_
#define NBLA_FUNCTION_INQ_CONVOLUTION_HPP_

#include <nbla/function/inq_affine.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(INQConvolution, int, const vector<int> &, const vector<int> &, const vector<int> &, int,
                              int, const vector<int> &, const string &, int);

// Inputs: x, weight (rewritten), indicator_fixedweights (int, rewritten), [bias].
template <typename T, typename T1>
class INQConvolution : public BaseFunction<int, const vector<int> &, const vector<int> &, const vector<int> &, int,
                                           int, const vector<int> &, const string &, int>,
                       protected InqState {
protected:
  int base_axis_;
  vector<int> pad_, stride_, dilation_;
  int group_;
  ConvShapes shapes_;

public:
  INQConvolution(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
                 const vector<int> &dilation, int group, int num_bits, const vector<int> &inq_iterations,
                 const string &selection_algorithm, int seed)
      : BaseFunction(ctx, base_axis, pad, stride, dilation, group, num_bits, inq_iterations, selection_algorithm,
                     seed),
        InqState(num_bits, inq_iterations, selection_algorithm, seed), base_axis_(base_axis), pad_(pad),
        stride_(stride), dilation_(dilation), group_(group) {}
  virtual ~INQConvolution() {}
  virtual shared_ptr<Function> copy() const {
    return create_INQConvolution(ctx_, base_axis_, pad_, stride_, dilation_, group_, num_bits_, inq_iterations_,
                                 selection_algorithm_, seed_);
  }
  virtual vector<dtypes> in_types() {
    return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T1>(), get_dtype<T>()};
  }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 3; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "INQConvolution"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  // inq_convolution.cpp:35-102
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    shapes_ = infer_conv_shapes(base_axis_, pad_, stride_, dilation_, group_, inputs[0], inputs[1],
                                inputs.size() == 4 ? inputs[3] : nullptr);
    base_axis_ = shapes_.base_axis;
    outputs[0]->reshape(shapes_.out_shape, true);
    this->setup_state(inputs[1], inputs[2]);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("INQConvolution"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("INQConvolution backward");
  }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 1 || i == 2; }
};

} // namespace nbla
#endif
