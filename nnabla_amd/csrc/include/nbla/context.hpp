// Execution context: ordered backend list, array class, device id
// (mirrors include/nbla/context.hpp:31-60).
#ifndef NBLA_CONTEXT_HPP_
#define NBLA_CONTEXT_HPP_

#include <nbla/common.hpp>

namespace nbla {

class NBLA_API Context {
public:
  explicit Context(const vector<string> &backend = {"cpu:float"}, const string &array_class = "CpuArray",
                   const string &device_id = "0");
  vector<string> backend;
  string array_class;
  string device_id;
  Context &set_backend(const vector<string> &backend);
  Context &set_array_class(const string &array_class);
  Context &set_device_id(const string &device_id);
  string to_string() const;
};

// Key used by registries that do not care about the backend list.
inline string get_array_key_from_context(const Context &ctx) { return ctx.device_id + ":" + ctx.array_class; }

} // namespace nbla
#endif
