// INQAffine: the class a "hip:float" implementation derives from.  Constructor, argument types, member
// names are those of include/nbla/function/inq_affine.hpp:76-147.
// This build has no CPU arithmetic: a generic *_impl method without a body of its own raises not_implemented.
#ifndef NBLA_FUNCTION_INQ_AFFINE_HPP_
#define NBLA_FUNCTION_INQ_AFFINE_HPP_

#include <nbla/cpu.hpp>
#include <nbla/function.hpp>
#include <nbla/function/no_cpu_impl.hpp>
#include <nbla/function_registry.hpp>

#include <random>

namespace nbla {

NBLA_REGISTER_FUNCTION_HEADER(INQAffine, int, int, const vector<int> &, const string &, int);

// Inputs: x, weight (rewritten), indicator_fixedweights (int, rewritten), [bias].
template <typename T, typename T1>
class INQAffine : public BaseFunction<int, int, const vector<int> &,
    const string &, int> {
protected:
  int base_axis_;
  int num_bits_;
  const vector<int> inq_iterations_;
  const string selection_algorithm_;
  int seed_;

  Variable old_weights_;
  Variable old_indicators_;
  int minibatch_counter_;
  std::mt19937 rgen_;
  std::bernoulli_distribution rdist_;

public:
  INQAffine(const Context &ctx, int base_axis, int num_bits, const vector<int> &inq_iterations,
        const string &selection_algorithm, int seed) : BaseFunction(ctx, base_axis, num_bits, inq_iterations,
        selection_algorithm, seed), base_axis_(base_axis), num_bits_(num_bits), inq_iterations_(inq_iterations),
        selection_algorithm_(selection_algorithm), seed_(seed), minibatch_counter_(0) {}
  virtual ~INQAffine() {}
  virtual shared_ptr<Function> copy() const { return create_INQAffine(ctx_, base_axis_, num_bits_, inq_iterations_,
      selection_algorithm_, seed_); }
  virtual vector<dtypes> in_types() { return vector<dtypes>{get_dtype<T>(), get_dtype<T>(), get_dtype<T1>(),
      get_dtype<T>()}; }
  virtual vector<dtypes> out_types() { return vector<dtypes>{get_dtype<T>()}; }
  virtual int min_inputs() { return 3; }
  virtual int min_outputs() { return 1; }
  virtual string name() { return "INQAffine"; }
  virtual vector<string> allowed_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }
  virtual bool grad_depends_output_data(int i, int o) const { return false; }

protected:
  virtual void setup_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("INQAffine"); }
  virtual void forward_impl(const Variables &, const Variables &) { NBLA_NO_CPU_IMPL("INQAffine"); }
  virtual void backward_impl(const Variables &, const Variables &, const vector<bool> &, const vector<bool> &) {
    NBLA_NO_CPU_IMPL("INQAffine backward");
  }
  virtual bool grad_depends_input_data_impl(int i, int j) const { return (i == 0 && j == 1) || (i == 1 && j == 0); }
  virtual bool overwrite_input_data_in_forward_impl(int i) const { return i == 1 || i == 2; }
};

} // namespace nbla
#endif
