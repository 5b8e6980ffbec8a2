// Backend lookup by the name in front of ':' in Context::backend[0]
// (mirrors include/nbla/backend_registry.hpp, src/nbla/backend_registry.cpp:34-55).
#ifndef NBLA_BACKEND_REGISTRY_HPP_
#define NBLA_BACKEND_REGISTRY_HPP_

#include <nbla/backend_base.hpp>
#include <nbla/context.hpp>

#include <functional>
#include <map>

namespace nbla {

class NBLA_API BackendUtils {
public:
  typedef std::function<BackendBase *(void)> BackendGetter;
  static void add_backend(const string &backend_name, BackendGetter backend_getter);
  static vector<string> array_classes(const Context ctx);
  static void _set_array_classes(const Context ctx, const vector<string> &a);
  static void register_array_class(const Context ctx, const string &name);
  static shared_ptr<Allocator> caching_allocator(const Context ctx);
  static shared_ptr<Allocator> naive_allocator(const Context ctx);
  static void free_unused_host_caches(const Context ctx);
  static void device_synchronize(const Context ctx);
  static void default_stream_synchronize(const Context ctx);
  static void create_lms_streams(const Context ctx);

private:
  static std::map<string, BackendGetter> &get_registry();
  static BackendBase *get_backend(const Context ctx);
};

#define NBLA_REGISTER_BACKEND(BACKEND_NAME, BACKEND_GETTER) ::nbla::BackendUtils::add_backend(BACKEND_NAME, BACKEND_GETTER)

} // namespace nbla
#endif
