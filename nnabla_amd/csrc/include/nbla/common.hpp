// Basic vocabulary types of the nbla core (mirrors include/nbla/common.hpp and
// include/nbla/dtypes.hpp of nnabla: same names, same enum values).
#ifndef NBLA_COMMON_HPP_
#define NBLA_COMMON_HPP_

#include <cstddef>
#include <cstdint>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#define NBLA_API __attribute__((visibility("default")))

namespace nbla {

using std::make_shared;
using std::shared_ptr;
using std::string;
using std::vector;

typedef vector<int64_t> Shape_t;
typedef int64_t Size_t;

// numpy-compatible dtype codes (dtypes.hpp:32-64)
enum class dtypes {
  BOOL = 0,
  BYTE,
  UBYTE,
  SHORT,
  USHORT,
  INT,
  UINT,
  LONG,
  ULONG,
  LONGLONG,
  ULONGLONG,
  FLOAT,
  DOUBLE,
  LONGDOUBLE,
  HALF = 23,
};

template <typename T> dtypes get_dtype();
template <> inline dtypes get_dtype<bool>() { return dtypes::BOOL; }
template <> inline dtypes get_dtype<signed char>() { return dtypes::BYTE; }
template <> inline dtypes get_dtype<unsigned char>() { return dtypes::UBYTE; }
template <> inline dtypes get_dtype<short>() { return dtypes::SHORT; }
template <> inline dtypes get_dtype<unsigned short>() { return dtypes::USHORT; }
template <> inline dtypes get_dtype<int>() { return dtypes::INT; }
template <> inline dtypes get_dtype<unsigned int>() { return dtypes::UINT; }
template <> inline dtypes get_dtype<long>() { return dtypes::LONG; }
template <> inline dtypes get_dtype<unsigned long>() { return dtypes::ULONG; }
template <> inline dtypes get_dtype<long long>() { return dtypes::LONGLONG; }
template <> inline dtypes get_dtype<unsigned long long>() { return dtypes::ULONGLONG; }
template <> inline dtypes get_dtype<float>() { return dtypes::FLOAT; }
template <> inline dtypes get_dtype<double>() { return dtypes::DOUBLE; }

NBLA_API size_t sizeof_dtype(dtypes dtype);
NBLA_API string dtype_to_string(dtypes dtype);

inline Size_t compute_size_by_shape(const Shape_t &shape, size_t axis = 0) {
  Size_t s = 1;
  for (size_t i = axis; i < shape.size(); ++i)
    s *= shape[i];
  return s;
}

inline Shape_t get_c_contiguous_strides(const Shape_t &shape) {
  Shape_t strides(shape.size(), 1);
  for (int i = (int)shape.size() - 2; i >= 0; --i)
    strides[i] = strides[i + 1] * shape[i + 1];
  return strides;
}

template <typename T> inline string string_join(const vector<T> &v, const string &delim) {
  std::ostringstream oss;
  for (size_t i = 0; i < v.size(); ++i) {
    if (i)
      oss << delim;
    oss << v[i];
  }
  return oss.str();
}


} // namespace nbla
#endif
