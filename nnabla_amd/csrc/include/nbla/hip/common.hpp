// Glue between the nbla host layer and the kernel library's C-ABI.
#ifndef NBLA_HIP_COMMON_HPP_
#define NBLA_HIP_COMMON_HPP_

#include <nbla/array.hpp>
#include <nbla/exception.hpp>

#include <nbla_hip_kernels.h>

namespace nbla {

// Turns a C-ABI status into the nbla::Exception the CPU class would have thrown for the same condition.
NBLA_API void hip_throw_on_error(int rc, const char *call, const char *func, const char *file, int line);
#define NBLA_HIP_CALL(expr)                                                                                            \
  do {                                                                                                                 \
    const int rc__ = (expr);                                                                                           \
    if (rc__ != 0)                                                                                                     \
      ::nbla::hip_throw_on_error(rc__, #expr, __func__, __FILE__, __LINE__);                                           \
  } while (0)

// "0", "1", ... -> device index (error_code::value for anything else).
NBLA_API int hip_device_index(const string &device_id);
// Makes the context's device current and initialises the kernel library for it.
NBLA_API int hip_set_device(const Context &ctx);

// A scratch buffer from the hip backend's caching allocator, released when it goes out of scope.
class NBLA_API HipWorkspace {
  ArrayPtr array_;
  size_t bytes_;

public:
  HipWorkspace(size_t bytes, const Context &ctx);
  void *pointer();
  size_t bytes() const { return bytes_; }
};

} // namespace nbla
#endif
