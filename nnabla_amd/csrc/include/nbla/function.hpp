// Function interface (mirrors include/nbla/function.hpp:65-477 and the protocol of src/nbla/function.cpp:27-174).
#ifndef NBLA_FUNCTION_HPP_
#define NBLA_FUNCTION_HPP_

#include <nbla/context.hpp>
#include <nbla/variable.hpp>

#include <tuple>

namespace nbla {

class NBLA_API Function {
  bool used_ = false;

public:
  typedef shared_ptr<Function> Ptr;

protected:
  Context ctx_;
  vector<shared_ptr<Shape_t>> in_shapes;
  vector<shared_ptr<Shape_t>> out_shapes;
  bool fall_back_func_ = false;
  bool called_setup_ = false;

public:
  explicit Function(const Context &ctx);
  virtual ~Function() = 0;
  Function(const Function &) = delete;
  Function &operator=(const Function &) = delete;

  // Picks the array class, checks arity, lets the implementation infer output shapes, memoises the shapes.
  void setup(const Variables &inputs, const Variables &outputs);
  // Re-runs setup when input shapes changed, then computes the outputs.
  void forward(const Variables &inputs, const Variables &outputs);
  void backward(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                const vector<bool> &accum);
  void setup_recompute(const Variables &inputs, const Variables &outputs);
  void recompute(const Variables &inputs, const Variables &outputs);

  Context context() const { return ctx_; }
  virtual vector<dtypes> in_types() = 0;
  virtual vector<dtypes> out_types() = 0;
  virtual int min_inputs() = 0;
  virtual int min_outputs() = 0;
  virtual string name() = 0;
  virtual vector<string> allowed_array_classes() = 0;
  virtual bool grad_depends_output_data(int i, int o) const { return true; }
  virtual bool grad_depends_input_data(int i, int j) const final { return grad_depends_input_data_impl(i, j); }
  virtual int inplace_data(int i) const { return NOT_INPLACE; }
  virtual int inplace_data_with(int i) const { NBLA_ERROR(error_code::not_implemented, "not in-place"); }
  virtual bool overwrite_input_data_in_forward(int i) const final { return overwrite_input_data_in_forward_impl(i); }
  // A function that keeps its inputs' buffers (Sink) tells the graph engine not to clear or zero them.
  virtual bool prohibit_clear_input_buffers() const { return false; }
  virtual bool prohibit_zero_input_grad() const { return false; }
  virtual bool need_setup_recompute(int o) const { return false; }
  virtual shared_ptr<Function> copy() const = 0;
  bool ask_if_used_and_use() {
    bool r = used_;
    used_ = true;
    return r;
  }
  static const int NOT_INPLACE = 0;
  static const int INPLACE_NOT_MODIFY = 1;
  static const int INPLACE = 2;

protected:
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) = 0;
  virtual void forward_impl(const Variables &inputs, const Variables &outputs) = 0;
  virtual void backward_impl(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                             const vector<bool> &accum) = 0;
  virtual void setup_recompute_impl(const Variables &inputs, const Variables &outputs) {}
  virtual void recompute_impl(const Variables &inputs, const Variables &outputs) { forward_impl(inputs, outputs); }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return true; }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return false; }
};
typedef Function::Ptr FunctionPtr;

// Stores the constructor arguments (what `copy()` and NNP serialisation read back).
template <typename... Args> class BaseFunction : public Function {
protected:
  std::tuple<typename std::remove_reference<Args>::type...> args_;

public:
  typedef BaseFunction<Args...> base_function_type;
  BaseFunction(const Context &ctx, Args... args) : Function(ctx), args_(args...) {}
  int num_args() { return sizeof...(Args); }
  const std::tuple<typename std::remove_reference<Args>::type...> &get_args() { return args_; }
};

// One-shot helper used by composite functions: setup + forward (src/nbla/imperative.cpp:66-69).
NBLA_API void execute(FunctionPtr f, const Variables &inputs, const Variables &outputs);

} // namespace nbla
#endif
