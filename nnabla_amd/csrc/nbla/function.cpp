// Function protocol, the per-function registries and the setup logic shared by the function headers.
#include <nbla/function.hpp>
#include <nbla/function/affine.hpp>
#include <nbla/function/binary_connect_affine.hpp>
#include <nbla/function/binary_connect_convolution.hpp>
#include <nbla/function/binary_weight_affine.hpp>
#include <nbla/function/binary_weight_convolution.hpp>
#include <nbla/function/convolution.hpp>
#include <nbla/function/fixed_point_quantize.hpp>
#include <nbla/function/inq_affine.hpp>
#include <nbla/function/inq_convolution.hpp>
#include <nbla/function/min_max_quantize.hpp>
#include <nbla/function/pow2_quantize.hpp>
#include <nbla/function/quantize_linear.hpp>
#include <nbla/function/range_recorder.hpp>

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
NBLA_REGISTER_FUNCTION_SOURCE(RangeRecorder, int, double, bool);

// ------------------------------------------------------------- shape inference
AffineShapes infer_affine_shapes(int base_axis, Variable *x, Variable *w, Variable *bias) {
  AffineShapes s;
  const Shape_t shape_data = x->shape();
  const Shape_t shape_weights = w->shape();
  NBLA_CHECK(shape_weights.size() >= 2, error_code::value, "Weights(inputs[1]) must be matrix or tensor.");
  refine_axis(base_axis, (int)x->ndim());
  s.base_axis = base_axis;
  NBLA_CHECK((size_t)base_axis < shape_data.size(), error_code::value,
             "Base_axis must be less than ndim of input data(inputs[0]). base_axis: %d >= ndim of input: %d.",
             base_axis, (int)shape_data.size());
  NBLA_CHECK(x->size(base_axis) == shape_weights[0], error_code::value,
             "Size of input data(inputs[0]) and weights(inputs[1]) mismatch. size of input: %ld != size of weights: %ld.",
             (long)x->size(base_axis), (long)shape_weights[0]);
  s.i_col = x->size(base_axis);
  s.i_row = s.i_col ? x->size() / s.i_col : 0;
  s.w_row = shape_weights[0];
  s.w_col = s.w_row ? w->size() / s.w_row : 0;
  for (int i = 0; i < base_axis; ++i)
    s.out_shape.push_back(shape_data[i]);
  for (size_t i = 1; i < shape_weights.size(); ++i)
    s.out_shape.push_back(shape_weights[i]);
  if (bias) {
    const Shape_t shape_bias = bias->shape();
    NBLA_CHECK(shape_bias.size() == shape_weights.size() - 1, error_code::value,
               "Length of bias(inputs[2]) and weights(inputs[1]) mismatch. bias length: %d != weights length-1: %d.",
               (int)shape_bias.size(), (int)shape_weights.size() - 1);
    for (size_t i = 0; i < shape_bias.size(); ++i)
      NBLA_CHECK(shape_bias[i] == shape_weights[i + 1], error_code::value,
                 "Shape of bias(inputs[2]) and weights(inputs[1]) mismatch.");
  }
  return s;
}

ConvShapes infer_conv_shapes(int base_axis, const vector<int> &pad, const vector<int> &stride,
                             const vector<int> &dilation, int group, Variable *x, Variable *w, Variable *bias) {
  ConvShapes s;
  const Shape_t shape_data = x->shape();
  const Shape_t shape_weights = w->shape();
  refine_axis(base_axis, (int)x->ndim());
  s.base_axis = base_axis;
  NBLA_CHECK((size_t)base_axis < shape_data.size() - 1, error_code::unclassified,
             "base_axis must be less than ndim - 1 of inputs[0]. base_axis: %d >= ndim of inputs[0] - 1: %d.",
             base_axis, (int)shape_data.size() - 1);
  const size_t spatial_dims = shape_data.size() - base_axis - 1;
  NBLA_CHECK(shape_weights.size() == 2 + spatial_dims, error_code::value, "Weights must be a tensor more than 3D.");
  s.spatial_dims = (int)spatial_dims;
  s.group = group;
  s.channels_i = shape_data[base_axis];
  s.channels_o = shape_weights[0];
  s.channels_g = shape_weights[1];
  NBLA_CHECK(group > 0 && s.channels_i % group == 0, error_code::value,
             "Number of input channel needs to be divisible by group. Input channel: %ld, group: %d.",
             (long)s.channels_i, group);
  NBLA_CHECK(s.channels_o % group == 0, error_code::value,
             "Number of output channel needs to be divisible by group. Output channel: %ld, group: %d.",
             (long)s.channels_o, group);
  NBLA_CHECK(s.channels_i / group == s.channels_g, error_code::value,
             "Number of grouped channel mismatch. Input: %ld != Weights[1]: %ld.", (long)(s.channels_i / group),
             (long)s.channels_g);
  NBLA_CHECK(pad.size() == spatial_dims, error_code::value, "pad size mismatch. pad size: %d != spatial dims: %d.",
             (int)pad.size(), (int)spatial_dims);
  NBLA_CHECK(stride.size() == spatial_dims, error_code::value,
             "stride size mismatch. stride size: %d != spatial dims: %d.", (int)stride.size(), (int)spatial_dims);
  NBLA_CHECK(dilation.size() == spatial_dims, error_code::value,
             "dilation size mismatch. dilation size: %d != spatial dims: %d.", (int)dilation.size(),
             (int)spatial_dims);
  s.inner_size_k = s.channels_g;
  s.outer = 1;
  s.out_shape = Shape_t(shape_data.size());
  for (int i = 0; i < base_axis; ++i) {
    s.out_shape[i] = shape_data[i];
    s.outer *= shape_data[i];
  }
  s.out_shape[base_axis] = s.channels_o;
  for (size_t i = 0; i < spatial_dims; ++i) {
    const int64_t kernel = shape_weights[2 + i];
    const int64_t in = shape_data[base_axis + 1 + i];
    const int64_t k = dilation[i] * (kernel - 1) + 1;
    const int64_t o = (in + 2 * pad[i] - k) / stride[i] + 1;
    NBLA_CHECK(o > 0 && in + 2 * pad[i] - k >= 0, error_code::value,
               "Invalid configuration of convolution at %d-th spatial dimension.  {input:%ld, kernel:%ld, pad:%d, "
               "stride:%d, dilation:%d}.",
               (int)i, (long)in, (long)kernel, pad[i], stride[i], dilation[i]);
    s.kernel.push_back(kernel);
    s.pad.push_back(pad[i]);
    s.stride.push_back(stride[i]);
    s.dilation.push_back(dilation[i]);
    s.spatial_i.push_back(in);
    s.spatial_o.push_back(o);
    s.inner_size_k *= kernel;
    s.out_shape[base_axis + 1 + i] = o;
  }
  if (bias) {
    NBLA_CHECK(bias->shape().size() == 1, error_code::value, "Bias(inputs[2]) must be a 1d tensor.");
    NBLA_CHECK(bias->shape()[0] == s.channels_o, error_code::value,
               "Shape of bias(inputs[2]) and weights(inputs[1]) mismatch. bias shape[0]: %ld != weights shape[0]: %ld.",
               (long)bias->shape()[0], (long)s.channels_o);
  }
  return s;
}

// -------------------------------------------------------------------- InqState
// Process-wide generator used when seed == -1 (the role of nnabla's RandomManager, seed 313).
static std::mt19937 &global_generator() {
  static std::mt19937 g(313);
  return g;
}

void InqState::setup_state(Variable *weights, Variable *indicators) {
  NBLA_CHECK(weights->shape().size() == indicators->shape().size(), error_code::value,
             "Indicators and weights must have same size. Ndim of weights: %d != ndim of indicators: %d.",
             (int)weights->shape().size(), (int)indicators->shape().size());
  NBLA_CHECK(weights->shape() == indicators->shape(), error_code::value,
             "Indicators and weights must have same size.");
  NBLA_CHECK(selection_algorithm_ == "largest_abs" || selection_algorithm_ == "random", error_code::value,
             "Provided value for selection algorithm not valid: %s. Valid values are \"largest_abs\" and \"random\".",
             selection_algorithm_.c_str());
  if (selection_algorithm_ == "random") {
    std::random_device rdev;
    rgen_ = std::mt19937(seed_ == -1 ? rdev() : (unsigned)seed_);
    rdist_ = std::bernoulli_distribution(0.5);
  }
  minibatch_counter_ = 0;
  old_weights_.reshape(weights->shape(), true);
  old_indicators_.reshape(weights->shape(), true);
  old_indicators_.data()->zero();
}

int InqState::current_step() const {
  if (std::find(inq_iterations_.begin(), inq_iterations_.end(), minibatch_counter_) == inq_iterations_.end())
    return 0;
  if (inq_iterations_.back() == minibatch_counter_)
    return 1;
  return selection_algorithm_ == "largest_abs" ? 2 : 3;
}

std::mt19937 &InqState::generator() { return seed_ == -1 ? global_generator() : rgen_; }

} // namespace nbla
