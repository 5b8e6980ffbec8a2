// Convolution (mirrors include/nbla/function/convolution.hpp): the plain product the quantized parametric layers
// run their quantized weights through.
#ifndef NBLA_FUNCTION_CONVOLUTION_HPP_
#define NBLA_FUNCTION_CONVOLUTION_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Convolution, int, const vector<int> &, const vector<int> &, const vector<int> &, int,
                              bool);

// Inputs: x, weight, [bias].
template <typename T>
class Convolution : public BaseFunction<int, const vector<int> &, const vector<int> &, const vector<int> &, int, bool> {
protected:
  int base_axis_;
  vector<int> pad_, stride_, dilation_;
  int group_;
  bool channel_last_;
  ConvShapes shapes_;

public:
  Convolution(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
              const vector<int> &dilation, int group, bool channel_last)
      : BaseFunction(ctx, base_axis, pad, stride, dilation, group, channel_last), base_axis_(base_axis), pad_(pad),
        stride_(stride), dilation_(dilation), group_(group), channel_last_(channel_last) {}
  virtual ~Convolution() {}
  virtual shared_ptr<Function> copy() const {
    return create_Convolution(ctx_, base_axis_, pad_, stride_, dilation_, group_, channel_last_);
  }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Convolution"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  // convolution.cpp:41-160
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    NBLA_CHECK(!channel_last_, error_code::not_implemented,
               "The passed argument channel_last_=true is not supported in Convolution.");
    shapes_ = infer_conv_shapes(base_axis_, pad_, stride_, dilation_, group_, inputs[0], inputs[1],
                                inputs.size() == 3 ? inputs[2] : nullptr);
    base_axis_ = shapes_.base_axis;
    outputs[0]->reshape(shapes_.out_shape, true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Convolution"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Convolution backward");
  }
};

} // namespace nbla
#endif
