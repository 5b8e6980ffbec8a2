// Concatenate: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/concatenate.hpp:27-88.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_CONCATENATE_HPP_
#define NBLA_FUNCTION_CONCATENATE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(Concatenate, int);

// Inputs: two or more arrays whose shapes differ along `axis` at most.
template <typename T> class Concatenate : public BaseFunction<int> {
protected:
  int axis_;
  int outer_size_, inner_total_size_;

public:
  Concatenate(const Context &ctx, int axis) : BaseFunction(ctx, axis), axis_(axis) {}
  virtual ~Concatenate() {}
  virtual shared_ptr<Function> copy() const { return create_Concatenate(ctx_, axis_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 2; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "Concatenate"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    // concatenate.cpp:29-58
    Shape_t shape = inputs[0]->shape();
    if (axis_ < 0)
      axis_ += (int)shape.size();
    NBLA_CHECK(axis_ >= 0 && axis_ < (int)shape.size(), error_code::value, "axis %d is out of range for %d dimensions.",
               axis_, (int)shape.size());
    inner_total_size_ = 0;
    for (Variables::size_type i = 0; i < inputs.size(); i++) {
      NBLA_CHECK(inputs[i]->shape().size() != 0, error_code::value, "input value(inputs[%d]) does not exist.", (int)i);
      inner_total_size_ += (int)inputs[i]->size(axis_);
      if (i >= 1) {
        NBLA_CHECK(inputs[i]->shape().size() == shape.size(), error_code::value, "Dimensions of inputs must match.");
        shape[axis_] += inputs[i]->shape()[axis_];
        for (Shape_t::size_type j = 0; j < shape.size(); j++)
          if ((int)j != axis_)
            NBLA_CHECK(inputs[i]->shape()[j] == shape[j], error_code::value,
                       "Dimensions of inputs must match. inputs[%d]->shape()[%d]: %d != inputs[0]->shape()[%d]: %d.",
                       (int)i, (int)j, (int)inputs[i]->shape()[j], (int)j, (int)shape[j]);
      }
    }
    outputs[0]->reshape(shape, true);
    outer_size_ = (int)(inputs[0]->size() / inputs[0]->size(axis_));
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("Concatenate"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("Concatenate backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return false; }
};

} // namespace nbla
#endif
