// Error reporting of the nbla core (mirrors include/nbla/exception.hpp:42-108).
#ifndef NBLA_EXCEPTION_HPP_
#define NBLA_EXCEPTION_HPP_

#include <nbla/common.hpp>

#include <cstdio>
#include <stdexcept>

namespace nbla {

enum class error_code {
  unclassified = 0,
  not_implemented,
  value,
  type,
  memory,
  io,
  os,
  target_specific,
  target_specific_async,
  runtime
};

NBLA_API string get_error_string(error_code code);

class NBLA_API Exception : public std::exception {
  error_code code_;
  string full_msg_, msg_, func_, file_;
  int line_;

public:
  Exception(error_code code, const string &msg, const string &func, const string &file, int line);
  virtual ~Exception() throw() {}
  virtual const char *what() const throw() { return full_msg_.c_str(); }
  error_code code() const { return code_; }
  const string &message() const { return msg_; }
};

template <typename... Args> string format_string(const string &fmt, Args... args) {
  int n = std::snprintf(nullptr, 0, fmt.c_str(), args...);
  if (n <= 0)
    return string();
  vector<char> buf(n + 1);
  std::snprintf(buf.data(), buf.size(), fmt.c_str(), args...);
  return string(buf.data(), n);
}
inline string format_string(const string &fmt) { return fmt; }

#define NBLA_ERROR(code, msg, ...)                                                                                     \
  throw ::nbla::Exception(code, ::nbla::format_string(msg, ##__VA_ARGS__), __func__, __FILE__, __LINE__)

#define NBLA_CHECK(condition, code, msg, ...)                                                                          \
  if (!(condition)) {                                                                                                  \
    /* the condition text is appended after formatting: it may itself contain '%' */                                  \
    throw ::nbla::Exception(code, ::nbla::string("Failed `" #condition "`: ") + ::nbla::format_string(msg, ##__VA_ARGS__), \
                            __func__, __FILE__, __LINE__);                                                             \
  }

} // namespace nbla
#endif
