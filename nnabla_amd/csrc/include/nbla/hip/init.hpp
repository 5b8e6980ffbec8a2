// Registration of the hip backend: arrays, synchronisers, and the "hip:float" Function implementations.
#ifndef NBLA_HIP_INIT_HPP_
#define NBLA_HIP_INIT_HPP_

#include <nbla/common.hpp>

namespace nbla {
// Idempotent and thread-safe; the counterpart of init_cpu() (src/nbla/init.cpp.tmpl:44-111).
NBLA_API void init_hip();
NBLA_API vector<string> hip_array_classes();
NBLA_API void hip_device_synchronize(const string &device);
NBLA_API int hip_get_device_count();
NBLA_API vector<string> hip_get_devices();
NBLA_API void hip_clear_memory_cache();
} // namespace nbla
#endif
