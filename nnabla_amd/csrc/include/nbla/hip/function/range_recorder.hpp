// "hip:float" implementations of Sink and the range recorders.
#ifndef NBLA_HIP_FUNCTION_RANGE_RECORDER_HPP_
#define NBLA_HIP_FUNCTION_RANGE_RECORDER_HPP_

#include <nbla/function/range_recorder.hpp>
#include <nbla/hip/hip.hpp>

namespace nbla {

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
