// INQAffine (mirrors include/nbla/function/inq_affine.hpp:76-147).
#ifndef NBLA_FUNCTION_INQ_AFFINE_HPP_
#define NBLA_FUNCTION_INQ_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function/utils_shapes.hpp>
#include <nbla/function_registry.hpp>

#include <algorithm>
#include <random>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(INQAffine, int, int, const vector<int> &, const string &, int);

// State and bookkeeping common to INQAffine and INQConvolution: the minibatch counter, the snapshot of weights
// and indicators, and the host-side generator of the "random" selection (inq_affine.hpp:86-92).
class NBLA_API InqState {
public:
  int num_bits_;
  vector<int> inq_iterations_;
  string selection_algorithm_;
  int seed_;
  int minibatch_counter_ = 0;
  Variable old_weights_, old_indicators_;
  std::mt19937 rgen_;
  std::bernoulli_distribution rdist_;
  InqState(int num_bits, const vector<int> &inq_iterations, const string &selection_algorithm, int seed)
      : num_bits_(num_bits), inq_iterations_(inq_iterations), selection_algorithm_(selection_algorithm), seed_(seed) {}
  // inq_affine.cpp:53-79
  void setup_state(Variable *weights, Variable *indicators);
  // The indicator update the current minibatch calls for (:104-113):
  // 0 none, 1 fix all, 2 largest_abs, 3 random.
  int current_step() const;
  std::mt19937 &generator();
};

// Inputs: x, weight (rewritten), indicator_fixedweights (int, rewritten), [bias].
template <typename T, typename T1>
class INQAffine : public BaseFunction<int, int, const vector<int> &, const string &, int>, protected InqState {
protected:
  int base_axis_;
  AffineShapes shapes_;

public:
  INQAffine(const Context &ctx, int base_axis, int num_bits, const vector<int> &inq_iterations,
            const string &selection_algorithm, int seed)
      : BaseFunction(ctx, base_axis, num_bits, inq_iterations, selection_algorithm, seed),
        InqState(num_bits, inq_iterations, selection_algorithm, seed), base_axis_(base_axis) {}
  virtual ~INQAffine() {}
  virtual shared_ptr<Function> copy() const {
    return create_INQAffine(ctx_, base_axis_, num_bits_, inq_iterations_, selection_algorithm_, seed_);
  }
  virtual vector<dtypes> in_types() {
    return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T1>(), get_dtype<T>()};
  }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 3; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "INQAffine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  // inq_affine.cpp:34-79
  virtual void setup_impl(const Variables &inputs, const Variables &outputs) {
    shapes_ = infer_affine_shapes(base_axis_, inputs[0], inputs[1], inputs.size() == 4 ? inputs[3] : nullptr);
    base_axis_ = shapes_.base_axis;
    outputs[0]->reshape(shapes_.out_shape, true);
    this->setup_state(inputs[1], inputs[2]);
  }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("INQAffine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("INQAffine backward");
  }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 1 || i == 2; }
};

} // namespace nbla
#endif
