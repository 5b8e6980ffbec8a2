// Array base, host arrays, and the array registries.
#include <nbla/array/cpu_array.hpp>
#include <nbla/array_registry.hpp>
#include <nbla/cpu.hpp>
#include <nbla/singleton_manager.hpp>

#include <cstring>

namespace nbla {

Array::Array(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem, const Size_t offset)
    : size_(size), dtype_(dtype), ctx_(ctx), mem_(mem), offset_(offset) {}
Array::~Array() {}
void Array::wait_event(const Context &, int) {}

// ------------------------------------------------------------ host conversions
namespace {

template <typename Ta, typename Tb> void convert(const void *src, void *dst, Size_t size) {
  const Ta *s = static_cast<const Ta *>(src);
  Tb *d = static_cast<Tb *>(dst);
  for (Size_t i = 0; i < size; ++i)
    d[i] = static_cast<Tb>(s[i]);
}

template <typename Ta> void convert_from(const void *src, void *dst, dtypes dst_dtype, Size_t size) {
  switch (dst_dtype) {
  case dtypes::BOOL: return convert<Ta, bool>(src, dst, size);
  case dtypes::BYTE: return convert<Ta, signed char>(src, dst, size);
  case dtypes::UBYTE: return convert<Ta, unsigned char>(src, dst, size);
  case dtypes::SHORT: return convert<Ta, short>(src, dst, size);
  case dtypes::USHORT: return convert<Ta, unsigned short>(src, dst, size);
  case dtypes::INT: return convert<Ta, int>(src, dst, size);
  case dtypes::UINT: return convert<Ta, unsigned int>(src, dst, size);
  case dtypes::LONG: return convert<Ta, long>(src, dst, size);
  case dtypes::ULONG: return convert<Ta, unsigned long>(src, dst, size);
  case dtypes::LONGLONG: return convert<Ta, long long>(src, dst, size);
  case dtypes::ULONGLONG: return convert<Ta, unsigned long long>(src, dst, size);
  case dtypes::FLOAT: return convert<Ta, float>(src, dst, size);
  case dtypes::DOUBLE: return convert<Ta, double>(src, dst, size);
  default:
    NBLA_ERROR(error_code::type, "Unsupported destination dtype %s.", dtype_to_string(dst_dtype).c_str());
  }
}

template <typename T> void fill_typed(void *dst, Size_t size, float value) {
  T *d = static_cast<T *>(dst);
  const T v = static_cast<T>(value);
  for (Size_t i = 0; i < size; ++i)
    d[i] = v;
}

} // namespace

void cpu_array_copy(const void *src, dtypes src_dtype, void *dst, dtypes dst_dtype, Size_t size) {
  if (src_dtype == dst_dtype) {
    std::memcpy(dst, src, size * sizeof_dtype(src_dtype));
    return;
  }
  switch (src_dtype) {
  case dtypes::BOOL: return convert_from<bool>(src, dst, dst_dtype, size);
  case dtypes::BYTE: return convert_from<signed char>(src, dst, dst_dtype, size);
  case dtypes::UBYTE: return convert_from<unsigned char>(src, dst, dst_dtype, size);
  case dtypes::SHORT: return convert_from<short>(src, dst, dst_dtype, size);
  case dtypes::USHORT: return convert_from<unsigned short>(src, dst, dst_dtype, size);
  case dtypes::INT: return convert_from<int>(src, dst, dst_dtype, size);
  case dtypes::UINT: return convert_from<unsigned int>(src, dst, dst_dtype, size);
  case dtypes::LONG: return convert_from<long>(src, dst, dst_dtype, size);
  case dtypes::ULONG: return convert_from<unsigned long>(src, dst, dst_dtype, size);
  case dtypes::LONGLONG: return convert_from<long long>(src, dst, dst_dtype, size);
  case dtypes::ULONGLONG: return convert_from<unsigned long long>(src, dst, dst_dtype, size);
  case dtypes::FLOAT: return convert_from<float>(src, dst, dst_dtype, size);
  case dtypes::DOUBLE: return convert_from<double>(src, dst, dst_dtype, size);
  default:
    NBLA_ERROR(error_code::type, "Unsupported source dtype %s.", dtype_to_string(src_dtype).c_str());
  }
}

void cpu_fill(void *dst, dtypes dtype, Size_t size, float value) {
  switch (dtype) {
  case dtypes::BOOL: return fill_typed<bool>(dst, size, value);
  case dtypes::BYTE: return fill_typed<signed char>(dst, size, value);
  case dtypes::UBYTE: return fill_typed<unsigned char>(dst, size, value);
  case dtypes::SHORT: return fill_typed<short>(dst, size, value);
  case dtypes::USHORT: return fill_typed<unsigned short>(dst, size, value);
  case dtypes::INT: return fill_typed<int>(dst, size, value);
  case dtypes::UINT: return fill_typed<unsigned int>(dst, size, value);
  case dtypes::LONG: return fill_typed<long>(dst, size, value);
  case dtypes::ULONG: return fill_typed<unsigned long>(dst, size, value);
  case dtypes::LONGLONG: return fill_typed<long long>(dst, size, value);
  case dtypes::ULONGLONG: return fill_typed<unsigned long long>(dst, size, value);
  case dtypes::FLOAT: return fill_typed<float>(dst, size, value);
  case dtypes::DOUBLE: return fill_typed<double>(dst, size, value);
  default:
    NBLA_ERROR(error_code::type, "Unsupported dtype %s.", dtype_to_string(dtype).c_str());
  }
}

// -------------------------------------------------------------------- CpuArray
CpuArray::CpuArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem,
                   const Size_t offset)
    : Array(size, dtype, ctx,
            mem ? mem : SingletonManager::get<Cpu>()->naive_allocator()->alloc(Array::size_as_bytes(size, dtype), ""),
            offset) {}
CpuArray::~CpuArray() {}

void CpuArray::copy_from(const Array *src_array) {
  NBLA_CHECK(src_array->size() == size_, error_code::unclassified, "Size mismatch.");
  cpu_array_copy(src_array->const_pointer<void>(), src_array->dtype(), pointer<void>(), dtype_, size_);
}
void CpuArray::zero() { std::memset(pointer<void>(), 0, size_ * sizeof_dtype(dtype_)); }
void CpuArray::fill(float value) { cpu_fill(pointer<void>(), dtype_, size_, value); }
Context CpuArray::filter_context(const Context &) { return Context({}, "CpuArray", ""); }

CpuCachedArray::CpuCachedArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem,
                               const Size_t offset)
    : CpuArray(size, dtype, ctx,
               mem ? mem
                   : SingletonManager::get<Cpu>()->caching_allocator()->alloc(Array::size_as_bytes(size, dtype), ""),
               offset) {}
CpuCachedArray::~CpuCachedArray() {}
Context CpuCachedArray::filter_context(const Context &) { return Context({}, "CpuCachedArray", ""); }

void synchronizer_cpu_array_cpu_array(Array *src, Array *dst, int) { dst->copy_from(src); }

// ------------------------------------------------------------------ registries
std::map<string, std::pair<ArrayCreator::Creator, ArrayCreator::FilterContext>> &ArrayCreator::registry() {
  static std::map<string, std::pair<Creator, FilterContext>> r;
  return r;
}
void ArrayCreator::add_creator(const string &name, Creator creator, FilterContext filter_context) {
  registry()[name] = {creator, filter_context};
}
Array *ArrayCreator::create(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem,
                            const Size_t offset) {
  auto it = registry().find(ctx.array_class);
  if (it == registry().end()) {
    vector<string> have = get_array_classes();
    NBLA_ERROR(error_code::unclassified, "'%s' could not be found in [%s]", ctx.array_class.c_str(),
               string_join(have, ", ").c_str());
  }
  return it->second.first(size, dtype, ctx, mem, offset);
}
Context ArrayCreator::filter_context(const Context &ctx) {
  auto it = registry().find(ctx.array_class);
  if (it == registry().end()) {
    vector<string> have = get_array_classes();
    NBLA_ERROR(error_code::unclassified, "'%s' could not be found in [%s]", ctx.array_class.c_str(),
               string_join(have, ", ").c_str());
  }
  return it->second.second(ctx);
}
vector<string> ArrayCreator::get_array_classes() {
  vector<string> out;
  for (auto &kv : registry())
    out.push_back(kv.first);
  return out;
}

std::map<std::pair<string, string>, ArraySynchronizer::Synchronizer> &ArraySynchronizer::registry() {
  static std::map<std::pair<string, string>, Synchronizer> r;
  return r;
}
void ArraySynchronizer::add_synchronizer(const string &src_class, const string &dst_class, Synchronizer s) {
  registry()[{src_class, dst_class}] = s;
}
void ArraySynchronizer::synchronize(const string &src_class, Array *src_array, const string &dst_class,
                                    Array *dst_array, int async_flags) {
  auto it = registry().find({src_class, dst_class});
  if (it == registry().end()) {
    vector<string> have;
    for (auto &kv : registry())
      have.push_back(kv.first.first + "-->" + kv.first.second);
    NBLA_ERROR(error_code::unclassified, "Unregistered synchronizer [%s-->%s]. Registered: [%s]", src_class.c_str(),
               dst_class.c_str(), string_join(have, ", ").c_str());
  }
  it->second(src_array, dst_array, async_flags);
}

std::map<string, string> &ArrayGroup::registry() {
  static std::map<string, string> r;
  return r;
}
void ArrayGroup::add_group(const string &array_class, const string &group_name) {
  registry()[array_class] = group_name;
}
string ArrayGroup::get_group(const string &array_class) {
  auto it = registry().find(array_class);
  NBLA_CHECK(it != registry().end(), error_code::unclassified, "'%s' belongs to no array group.", array_class.c_str());
  return it->second;
}

} // namespace nbla
