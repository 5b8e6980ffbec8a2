// Output shape of a two-input element-wise function with broadcasting: the checks and the shape of
// BaseTransformBinary::setup_impl, include/nbla/function/utils/base_transform_binary.hpp:58-86 (the strides it goes on
// to compute are worked out by the kernel library from the two shapes).
#ifndef NBLA_FUNCTION_UTILS_BASE_TRANSFORM_BINARY_HPP_
#define NBLA_FUNCTION_UTILS_BASE_TRANSFORM_BINARY_HPP_

#include <nbla/exception.hpp>
#include <nbla/variable.hpp>

#include <algorithm>

namespace nbla {

inline void transform_binary_setup(const Variables &inputs, const Variables &outputs, bool inplace, const string &name) {
  const Size_t ndim = inputs[0]->ndim();
  NBLA_CHECK(ndim == inputs[1]->ndim(), error_code::value,
             "Dimensions of inputs must match. inputs[0]: %d != inputs[1]: %d.", (int)ndim, (int)inputs[1]->ndim());
  const Shape_t s0 = inputs[0]->shape(), s1 = inputs[1]->shape();
  Shape_t oshape(ndim);
  for (Size_t i = 0; i < ndim; ++i) {
    if (s0[i] != s1[i]) {
      NBLA_CHECK(std::min(s0[i], s1[i]) == 1, error_code::value, "Broadcast dimension must be one. shape[%d]: %d.",
                 (int)i, (int)std::min(s0[i], s1[i]));
    }
    oshape[i] = std::max(s0[i], s1[i]);
  }
  outputs[0]->reshape(oshape, true);
  // (the in-place form, :75-82, is obsolete in the reference and never requested by this build's callers)
  NBLA_CHECK(!inplace, error_code::not_implemented, "%s: the in-place form is not part of this build.", name.c_str());
}

} // namespace nbla
#endif
