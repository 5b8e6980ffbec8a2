// The generic Function classes of this build carry declarations only; their arithmetic exists in the "hip:float"
// implementations.  (Not part of nnabla's interface: no file outside nbla/function/ includes this.)
#ifndef NBLA_FUNCTION_NO_CPU_IMPL_HPP_
#define NBLA_FUNCTION_NO_CPU_IMPL_HPP_

#include <nbla/exception.hpp>

#define NBLA_NO_CPU_IMPL(NAME)                                                                                         \
  NBLA_ERROR(::nbla::error_code::not_implemented,                                                                      \
             NAME " has no CPU implementation in this build; create it with a 'hip:float' context.")

#endif
