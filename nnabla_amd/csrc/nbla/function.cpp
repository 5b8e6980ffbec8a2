// Function protocol, the per-function registries and the process-wide random generator.
#include <nbla/function.hpp>
#include <nbla/function/add2.hpp>
#include <nbla/function/div2.hpp>
#include <nbla/function/mul2.hpp>
#include <nbla/function/pow2.hpp>
#include <nbla/function/sub2.hpp>
#include <nbla/function/affine.hpp>
#include <nbla/function/binary_connect_affine.hpp>
#include <nbla/function/binary_connect_convolution.hpp>
#include <nbla/function/binary_weight_affine.hpp>
#include <nbla/function/binary_weight_convolution.hpp>
#include <nbla/function/concatenate.hpp>
#include <nbla/function/convolution.hpp>
#include <nbla/function/dequantize_linear.hpp>
#include <nbla/function/fixed_point_quantize.hpp>
#include <nbla/function/inq_affine.hpp>
#include <nbla/function/inq_convolution.hpp>
#include <nbla/function/min_max_quantize.hpp>
#include <nbla/function/pow2_quantize.hpp>
#include <nbla/function/prune.hpp>
#include <nbla/function/quantize_linear.hpp>
#include <nbla/function/relu.hpp>
#include <nbla/function/sink.hpp>
#include <nbla/random_manager.hpp>

#include <algorithm>

namespace nbla {

Function::Function(const Context &ctx) : ctx_(ctx) {}
Function::~Function() {}

// src/nbla/function.cpp:27-72
void Function::setup(const Variables &inputs, const Variables &outputs) {
  if (fall_back_func_) {
    // not used by this build
  }
  // The context's array class is used when the function allows it, else the function's default.
  const vector<string> allowed = this->allowed_array_classes();
  NBLA_CHECK(!allowed.empty(), error_code::value, "%s allows no array class.", this->name().c_str());
  if (std::find(allowed.begin(), allowed.end(), ctx_.array_class) == allowed.end())
    ctx_.array_class = allowed[0];
  NBLA_CHECK((int)inputs.size() >= this->min_inputs(), error_code::value,
             "%s needs at least %d inputs (given %d).", this->name().c_str(), this->min_inputs(), (int)inputs.size());
  NBLA_CHECK((int)outputs.size() >= this->min_outputs(), error_code::value,
             "%s needs at least %d outputs (given %d).", this->name().c_str(), this->min_outputs(),
             (int)outputs.size());
  this->setup_impl(inputs, outputs);
  in_shapes.clear();
  out_shapes.clear();
  for (Variable *v : inputs)
    in_shapes.push_back(make_shared<Shape_t>(v->shape()));
  for (Variable *v : outputs)
    out_shapes.push_back(make_shared<Shape_t>(v->shape()));
  called_setup_ = true;
}

namespace {
bool shapes_match(const vector<shared_ptr<Shape_t>> &memo, const Variables &vars) {
  if (memo.size() != vars.size())
    return false;
  for (size_t i = 0; i < vars.size(); ++i)
    if (*memo[i] != vars[i]->shape())
      return false;
  return true;
}
} // namespace

// src/nbla/function.cpp:107-123
void Function::forward(const Variables &inputs, const Variables &outputs) {
  NBLA_CHECK(called_setup_, error_code::unclassified, "%s: setup() must be called before forward().",
             this->name().c_str());
  if (!shapes_match(in_shapes, inputs) || !shapes_match(out_shapes, outputs))
    this->setup(inputs, outputs); // inputs were reshaped since the last setup
  this->forward_impl(inputs, outputs);
}

void Function::backward(const Variables &inputs, const Variables &outputs, const vector<bool> &propagate_down,
                        const vector<bool> &accum) {
  NBLA_CHECK(called_setup_, error_code::unclassified, "%s: setup() must be called before backward().",
             this->name().c_str());
  this->backward_impl(inputs, outputs, propagate_down, accum);
}

void Function::setup_recompute(const Variables &inputs, const Variables &outputs) {
  this->setup_recompute_impl(inputs, outputs);
}
void Function::recompute(const Variables &inputs, const Variables &outputs) { this->recompute_impl(inputs, outputs); }

void execute(FunctionPtr f, const Variables &inputs, const Variables &outputs) {
  f->setup(inputs, outputs);
  f->forward(inputs, outputs);
}

// ------------------------------------------------------------------ registries
NBLA_REGISTER_FUNCTION_SOURCE(FixedPointQuantize, bool, int, float, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Pow2Quantize, bool, bool, int, int, bool);
NBLA_REGISTER_FUNCTION_SOURCE(MinMaxQuantize, float, bool, bool, bool, float);
NBLA_REGISTER_FUNCTION_SOURCE(BinaryWeightAffine, int, float);
NBLA_REGISTER_FUNCTION_SOURCE(BinaryConnectAffine, int, float);
NBLA_REGISTER_FUNCTION_SOURCE(BinaryWeightConvolution, int, const vector<int> &, const vector<int> &,
                              const vector<int> &, int, float);
NBLA_REGISTER_FUNCTION_SOURCE(BinaryConnectConvolution, int, const vector<int> &, const vector<int> &,
                              const vector<int> &, int, float);
NBLA_REGISTER_FUNCTION_SOURCE(INQAffine, int, int, const vector<int> &, const string &, int);
NBLA_REGISTER_FUNCTION_SOURCE(INQConvolution, int, const vector<int> &, const vector<int> &, const vector<int> &, int,
                              int, const vector<int> &, const string &, int);
NBLA_REGISTER_FUNCTION_SOURCE(Affine, int);
NBLA_REGISTER_FUNCTION_SOURCE(ReLU, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Convolution, int, const vector<int> &, const vector<int> &, const vector<int> &, int, bool);
NBLA_REGISTER_FUNCTION_SOURCE(QuantizeLinear, const string &, bool, int);
NBLA_REGISTER_FUNCTION_SOURCE(DequantizeLinear);
NBLA_REGISTER_FUNCTION_SOURCE(Prune, float);
NBLA_REGISTER_FUNCTION_SOURCE(Sink, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Add2, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Sub2, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Pow2, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Mul2, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Div2, bool);
NBLA_REGISTER_FUNCTION_SOURCE(Concatenate, int);

// ----------------------------------------------------------------- RandomManager
RandomManager::RandomManager() : rgen_(313), seed_(313), count_(0) {}
RandomManager::~RandomManager() {}
std::mt19937 &RandomManager::get_rand_generator() { return rgen_; }
unsigned int RandomManager::get_seed() const { return seed_; }
void RandomManager::set_seed(unsigned int seed) {
  seed_ = seed;
  rgen_ = std::mt19937(seed);
  ++count_;
}
int RandomManager::get_count() const { return count_; }

} // namespace nbla
