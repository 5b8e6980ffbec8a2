// Registration of the host backend and host array classes (mirrors include/nbla/init.hpp,
// src/nbla/init.cpp.tmpl:44-111 without the cpu:float Function registrations: this build ships no CPU compute).
#ifndef NBLA_INIT_HPP_
#define NBLA_INIT_HPP_

#include <nbla/common.hpp>

namespace nbla {
NBLA_API void init_cpu();
NBLA_API void clear_all_singletons();
NBLA_API vector<string> cpu_array_classes();
} // namespace nbla
#endif
