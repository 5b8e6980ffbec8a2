// Sink: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/sink.hpp:36-82.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_SINK_HPP_
#define NBLA_FUNCTION_SINK_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Sink, bool);

// Inputs: any number of graph outputs.
template <typename T> class Sink : public BaseFunction<bool> {
protected:
  bool one_input_grad_;

public:
  Sink(const Context &ctx, bool one_input_grad) : BaseFunction(ctx, one_input_grad), one_input_grad_(one_input_grad) {}
  virtual ~Sink() {}
  virtual shared_ptr<Function> copy() const { return create_Sink(ctx_, one_input_grad_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 1; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Sink"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool prohibit_clear_input_buffers() const { return true; }
  virtual bool prohibit_zero_input_grad() const { return true; }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // sink.cpp:25-28
    outputs[0]->reshape({}, true);
  }
  // sink.cpp:30-33: nothing to compute
  virtual void forward_impl(const Variables &, const Variables &) {}
  // sink.cpp:35-48: seeds the gradients of the graph outputs it joins with ones
  virtual void backward_impl(const Variables &inputs, const Variables &, const vector<bool> &, const vector<bool> &) {
    if (!one_input_grad_)
      return;
    for (auto inp : inputs)
      inp->grad()->fill(1);
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

} // namespace nbla
#endif
