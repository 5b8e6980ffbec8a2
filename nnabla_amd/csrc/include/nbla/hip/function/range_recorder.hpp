// Sink and the range recorders of quantization-aware training on the hip backend.
//
// RangeRecorder is this extension's own function: nnabla writes the five recorders as PythonFunctions
// (python/src/nnabla/utils/qnn.py:42-560) and has no registry entry for them.  Here one registry function carries
// all five and reports the reference class's name, so that graph converters find them by the same type names.  Its
// registry (NBLA_REGISTER_FUNCTION_SOURCE) lives in the extension too.
#ifndef NBLA_HIP_FUNCTION_RANGE_RECORDER_HPP_
#define NBLA_HIP_FUNCTION_RANGE_RECORDER_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/sink.hpp>
#include <nbla/function_registry.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(RangeRecorder, int, double, bool);

// inputs: x, [m,] M; output: y = x.  mode: 0 MinMaxMinMaxRecorder, 1 AbsMaxRecorder, 2 MinMaxMvaRecorder,
// 3 MaxMaxRecorder, 4 MaxMvaRecorder.
template <typename T> class RangeRecorder : public BaseFunction<int, double, bool> {
protected:
  int mode_;
  double decay_; // the Python float of the reference's constructors
  bool training_;

public:
  RangeRecorder(const Context &ctx, int mode, double decay, bool training)
      : BaseFunction(ctx, mode, decay, training), mode_(mode), decay_(decay), training_(training) {
    NBLA_CHECK(mode >= 0 && mode <= 4, error_code::value, "RangeRecorder: unknown mode %d.", mode);
  }
  virtual ~RangeRecorder() {}
  virtual shared_ptr<Function> copy() const { return create_RangeRecorder(ctx_, mode_, decay_, training_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>(two_sided() ? 3 : 2, get_dtype<T>()); }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return two_sided() ? 3 : 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() {
    static const char *names[] = {"MinMaxMinMaxRecorder", "AbsMaxRecorder", "MinMaxMvaRecorder", "MaxMaxRecorder",
                                  "MaxMvaRecorder"};
    return names[mode_];
  }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }
  bool two_sided() const { return mode_ == 0 || mode_ == 2; }

protected:
  // the setup_impl of each recorder class: qnn.py:58-71, :164-176, :273-287, :397-409, :496-507
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    const size_t want = two_sided() ? 3 : 2;
    NBLA_CHECK(inputs.size() == want, error_code::value, "len(inputs) must be %d; data%s.", (int)want,
               two_sided() ? ", min, max" : ", max");
    for (size_t i = 1; i < want; ++i) {
      NBLA_CHECK(inputs[i]->ndim() == inputs[0]->ndim(), error_code::value,
                 "ndim of the recorded statistics must be same as ndim of data.");
      NBLA_CHECK(inputs[i]->size() == 1, error_code::value,
                 "Any dimension of the shape of the recorded statistics must be 1.");
    }
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) {
    NBLA_ERROR(error_code::not_implemented, "RangeRecorder has a 'hip:float' implementation only.");
  }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_ERROR(error_code::not_implemented, "RangeRecorder has a 'hip:float' implementation only.");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

template <typename T> class SinkHip : public Sink<T> {
public:
  SinkHip(const Context &ctx, bool one_input_grad) : Sink<T>(ctx, one_input_grad) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }
};

template <typename T> class RangeRecorderHip : public RangeRecorder<T> {
public:
  RangeRecorderHip(const Context &ctx, int mode, double decay, bool training)
      : RangeRecorder<T>(ctx, mode, decay, training) {}
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }

protected:
  virtual void forward_impl(const Variables &inputs, const Variables &outputs);
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum);
};

} // namespace nbla
#endif
