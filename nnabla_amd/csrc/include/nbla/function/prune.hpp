// Prune: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/prune.hpp:36-80.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_PRUNE_HPP_
#define NBLA_FUNCTION_PRUNE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Prune, float);

// Inputs: x.
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

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // prune.cpp:27-37
    NBLA_CHECK(rate_ >= 0 && rate_ <= 1, error_code::value, "Rate %f must be in [0, 1].", rate_);
    const int x_size = (int)inputs[0]->size();
    thresh_idx_ = (int)((x_size - 1) * this->rate_);
    outputs[0]->reshape(inputs[0]->shape(), true);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Prune"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Prune backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

} // namespace nbla
#endif
