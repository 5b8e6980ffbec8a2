// dtype tables, Context, Exception and SingletonManager.
#include <nbla/common.hpp>
#include <nbla/context.hpp>
#include <nbla/exception.hpp>
#include <nbla/singleton_manager.hpp>

namespace nbla {

size_t sizeof_dtype(dtypes dtype) {
  switch (dtype) {
  case dtypes::BOOL:
  case dtypes::BYTE:
  case dtypes::UBYTE:
    return 1;
  case dtypes::SHORT:
  case dtypes::USHORT:
  case dtypes::HALF:
    return 2;
  case dtypes::INT:
  case dtypes::UINT:
  case dtypes::FLOAT:
    return 4;
  case dtypes::LONG:
  case dtypes::ULONG:
  case dtypes::LONGLONG:
  case dtypes::ULONGLONG:
  case dtypes::DOUBLE:
    return 8;
  case dtypes::LONGDOUBLE:
    return sizeof(long double);
  }
  NBLA_ERROR(error_code::type, "Unsupported type: %d", (int)dtype);
}

string dtype_to_string(dtypes dtype) {
  switch (dtype) {
  case dtypes::BOOL: return "BOOL";
  case dtypes::BYTE: return "BYTE";
  case dtypes::UBYTE: return "UBYTE";
  case dtypes::SHORT: return "SHORT";
  case dtypes::USHORT: return "USHORT";
  case dtypes::INT: return "INT";
  case dtypes::UINT: return "UINT";
  case dtypes::LONG: return "LONG";
  case dtypes::ULONG: return "ULONG";
  case dtypes::LONGLONG: return "LONGLONG";
  case dtypes::ULONGLONG: return "ULONGLONG";
  case dtypes::FLOAT: return "FLOAT";
  case dtypes::DOUBLE: return "DOUBLE";
  case dtypes::LONGDOUBLE: return "LONGDOUBLE";
  case dtypes::HALF: return "HALF";
  }
  return "UNKNOWN";
}

// ------------------------------------------------------------------- Context
Context::Context(const vector<string> &backend, const string &array_class, const string &device_id)
    : backend(backend), array_class(array_class), device_id(device_id) {}
Context &Context::set_backend(const vector<string> &b) {
  backend = b;
  return *this;
}
Context &Context::set_array_class(const string &a) {
  array_class = a;
  return *this;
}
Context &Context::set_device_id(const string &d) {
  device_id = d;
  return *this;
}
string Context::to_string() const {
  return "Context(backend=[" + string_join(backend, ", ") + "], array_class='" + array_class + "', device_id='" +
         device_id + "')";
}

// ----------------------------------------------------------------- Exception
string get_error_string(error_code code) {
  switch (code) {
  case error_code::unclassified: return "unclassified";
  case error_code::not_implemented: return "not_implemented";
  case error_code::value: return "value";
  case error_code::type: return "type";
  case error_code::memory: return "memory";
  case error_code::io: return "io";
  case error_code::os: return "os";
  case error_code::target_specific: return "target_specific";
  case error_code::target_specific_async: return "target_specific_async";
  case error_code::runtime: return "runtime";
  }
  return "unknown";
}

Exception::Exception(error_code code, const string &msg, const string &func, const string &file, int line)
    : code_(code), msg_(msg), func_(func), file_(file), line_(line) {
  std::ostringstream ss;
  ss << get_error_string(code_) << " error in " << func_ << std::endl
     << file_ << ":" << line_ << std::endl
     << msg_ << std::endl;
  full_msg_ = ss.str();
}

// ---------------------------------------------------------- SingletonManager
SingletonManager &SingletonManager::get_self() {
  static SingletonManager *self = new SingletonManager(); // intentionally leaked: outlives static destructors
  return *self;
}

void SingletonManager::clear() {
  SingletonManager &self = get_self();
  std::lock_guard<std::recursive_mutex> lock(self.mtx_);
  for (auto it = self.order_.rbegin(); it != self.order_.rend(); ++it) {
    auto obj = self.objects_.find(*it);
    if (obj != self.objects_.end())
      obj->second.second(obj->second.first);
  }
  self.objects_.clear();
  self.order_.clear();
}

} // namespace nbla
