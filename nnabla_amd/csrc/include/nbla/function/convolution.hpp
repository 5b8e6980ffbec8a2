// Convolution: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/convolution.hpp:68-150.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_CONVOLUTION_HPP_
#define NBLA_FUNCTION_CONVOLUTION_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Convolution, int, const vector<int> &, const vector<int> &, const vector<int> &, int,
    bool);

// Inputs: x, weight, [bias].
template <typename T>
class Convolution : public BaseFunction<int, const vector<int> &, const vector<int> &,
    const vector<int> &, int, bool> {
protected:
  int base_axis_;
  vector<int> pad_;
  vector<int> stride_;
  vector<int> dilation_;
  int group_;
  bool channel_last_;
  vector<int> kernel_;
  Size_t channels_i_, channels_o_, channels_g_;
  vector<int> spatial_shape_i_;
  vector<int> spatial_shape_o_;
  int spatial_dims_;
  Size_t outer_size_;
  Size_t inner_size_i_;
  Size_t inner_size_o_;
  Size_t inner_size_k_;

public:
  Convolution(const Context &ctx, int base_axis, const vector<int> &pad, const vector<int> &stride,
        const vector<int> &dilation, int group, bool channel_last) : BaseFunction(ctx, base_axis, pad, stride,
        dilation, group, channel_last), base_axis_(base_axis), pad_(pad), stride_(stride), dilation_(dilation),
        group_(group), channel_last_(channel_last) {}
  virtual ~Convolution() {}
  virtual shared_ptr<Function> copy() const { return create_Convolution(ctx_, base_axis_, pad_, stride_, dilation_,
      group_, channel_last_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Convolution"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Convolution"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Convolution"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Convolution backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return (i == 0 && j == 1) || (i == 1 && j == 0); }
};

} // namespace nbla
#endif
