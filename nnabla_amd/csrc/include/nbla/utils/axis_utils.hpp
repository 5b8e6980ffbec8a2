// Axis arguments that may count from the end (mirrors include/nbla/utils/axis_utils.hpp:23-31).
#ifndef NBLA_UTILS_AXIS_UTILS_HPP_
#define NBLA_UTILS_AXIS_UTILS_HPP_

#include <nbla/exception.hpp>

namespace nbla {

// -ndim <= axis < ndim; a negative axis becomes axis + ndim.
inline void refine_axis(int &axis, int ndim) {
  NBLA_CHECK(axis < ndim && ndim + axis >= 0, error_code::value,
             "axis must be in the range of [-ndim, ndim). axis : %d, ndim: %d.", axis, ndim);
  if (axis < 0)
    axis += ndim;
}

} // namespace nbla
#endif
