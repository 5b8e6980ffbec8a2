// What a backend singleton provides (mirrors include/nbla/backend_base.hpp:32-91).
#ifndef NBLA_BACKEND_BASE_HPP_
#define NBLA_BACKEND_BASE_HPP_

#include <nbla/memory/allocator.hpp>

namespace nbla {

class NBLA_API BackendBase {
public:
  virtual ~BackendBase() {}
  // Array classes this backend's functions can work on; entry 0 is the default.
  virtual vector<string> array_classes() const = 0;
  virtual void _set_array_classes(const vector<string> &a) = 0;
  virtual void register_array_class(const string &name) = 0;
  virtual shared_ptr<Allocator> caching_allocator() = 0;
  virtual shared_ptr<Allocator> naive_allocator() = 0;
  virtual void free_unused_host_caches() = 0;
  virtual void device_synchronize(const string &device) = 0;
  virtual void default_stream_synchronize(const string &device) = 0;
  virtual void create_lms_streams(int device = -1) = 0;
};

} // namespace nbla
#endif
