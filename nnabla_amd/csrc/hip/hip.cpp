// The hip backend: error translation, device memory, device arrays, synchronisers, the backend singleton.
#include <nbla/array/cpu_array.hpp>
#include <nbla/array_registry.hpp>
#include <nbla/backend_registry.hpp>
#include <nbla/cpu.hpp>
#include <nbla/hip/array.hpp>
#include <nbla/hip/common.hpp>
#include <nbla/hip/hip.hpp>
#include <nbla/hip/init.hpp>
#include <nbla/hip/memory.hpp>
#include <nbla/memory/caching_allocator_with_buckets.hpp>
#include <nbla/memory/naive_allocator.hpp>

#include <cstdlib>

namespace nbla {

void hip_throw_on_error(int rc, const char *call, const char *func, const char *file, int line) {
  error_code code = error_code::target_specific;
  switch (rc) {
  case NBLA_HIP_ERR_NOT_IMPLEMENTED: code = error_code::not_implemented; break;
  case NBLA_HIP_ERR_VALUE: code = error_code::value; break;
  case NBLA_HIP_ERR_MEMORY: code = error_code::memory; break;
  case NBLA_HIP_ERR_RUNTIME: code = error_code::runtime; break;
  default: break;
  }
  throw Exception(code, format_string("%s (in %s, status %d)", nbla_hip_last_error(), call, rc), func, file, line);
}

int hip_device_index(const string &device_id) {
  char *end = nullptr;
  const long v = std::strtol(device_id.c_str(), &end, 10);
  NBLA_CHECK(!device_id.empty() && end && *end == '\0' && v >= 0, error_code::value,
             "Invalid device id '%s' for the hip backend.", device_id.c_str());
  return (int)v;
}

int hip_set_device(const Context &ctx) {
  const int dev = hip_device_index(ctx.device_id);
  NBLA_HIP_CALL(nbla_hip_init(dev));
  return dev;
}

HipWorkspace::HipWorkspace(size_t bytes, const Context &ctx) : bytes_(bytes ? bytes : 256) {
  Context c = ctx;
  c.array_class = "HipCachedArray";
  array_ = ArrayPtr(ArrayCreator::create((Size_t)bytes_, dtypes::BYTE, c));
}
void *HipWorkspace::pointer() { return array_->pointer<void>(); }

// ------------------------------------------------------------------- HipMemory
HipMemory::HipMemory(size_t bytes, const string &device_id) : Memory(bytes, device_id) {}
HipMemory::HipMemory(size_t bytes, const string &device_id, void *ptr) : Memory(bytes, device_id) { ptr_ = ptr; }
HipMemory::~HipMemory() {}

bool HipMemory::alloc_impl() {
  const int dev = hip_device_index(this->device_id());
  void *p = nullptr;
  if (nbla_hip_malloc(&p, bytes_, dev) != 0)
    return false;
  ptr_ = p;
  // Every fragment of this allocation shares the owner; the last one to go returns it to the device.
  root_ = shared_ptr<void>(p, [dev](void *q) { nbla_hip_free(q, dev); });
  return true;
}
shared_ptr<Memory> HipMemory::divide_impl(size_t second_start) {
  HipMemory *second = new HipMemory(bytes_ - second_start, this->device_id(), static_cast<char *>(ptr_) + second_start);
  second->root_ = root_;
  return shared_ptr<Memory>(second);
}
void HipMemory::merge_next_impl(Memory *) {}
void HipMemory::merge_prev_impl(Memory *from) { ptr_ = from->pointer(); }

// -------------------------------------------------------------------- HipArray
HipArray::HipArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem,
                   const Size_t offset)
    : Array(size, dtype, ctx,
            mem ? mem
                : SingletonManager::get<Hip>()->naive_allocator()->alloc(Array::size_as_bytes(size, dtype),
                                                                         ctx.device_id),
            offset),
      device_(hip_device_index(ctx.device_id)) {}
HipArray::~HipArray() {}

void HipArray::copy_from(const Array *src_array) {
  NBLA_CHECK(src_array->size() == size_, error_code::unclassified, "Size mismatch.");
  hip_set_device(ctx_);
  NBLA_HIP_CALL(nbla_hip_cast(src_array->const_pointer<void>(), (int)src_array->dtype(), pointer<void>(), (int)dtype_,
                              (size_t)size_, nullptr));
}
void HipArray::zero() {
  hip_set_device(ctx_);
  NBLA_HIP_CALL(nbla_hip_fill(pointer<void>(), (int)dtype_, (size_t)size_, 0.0f, nullptr));
}
void HipArray::fill(float value) {
  hip_set_device(ctx_);
  NBLA_HIP_CALL(nbla_hip_fill(pointer<void>(), (int)dtype_, (size_t)size_, value, nullptr));
}
Context HipArray::filter_context(const Context &ctx) { return Context({}, "HipArray", ctx.device_id); }

HipCachedArray::HipCachedArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem,
                               const Size_t offset)
    : HipArray(size, dtype, ctx,
               mem ? mem
                   : SingletonManager::get<Hip>()->caching_allocator()->alloc(Array::size_as_bytes(size, dtype),
                                                                              ctx.device_id),
               offset) {}
HipCachedArray::~HipCachedArray() {}
Context HipCachedArray::filter_context(const Context &ctx) { return Context({}, "HipCachedArray", ctx.device_id); }

// ---------------------------------------------------------------- synchronisers
// Device -> host.  With a dtype change the conversion runs on the device into a scratch array first.
void synchronizer_hip_array_cpu_array(Array *src, Array *dst, int) {
  NBLA_CHECK(src->size() == dst->size(), error_code::unclassified, "Size mismatch.");
  hip_set_device(src->context());
  if (src->size() == 0)
    return;
  if (src->dtype() == dst->dtype()) {
    NBLA_HIP_CALL(nbla_hip_memcpy(dst->pointer<void>(), src->const_pointer<void>(),
                                  (size_t)src->size() * sizeof_dtype(src->dtype()), 2, nullptr));
    return;
  }
  Context c = src->context();
  c.array_class = "HipCachedArray";
  ArrayPtr tmp(ArrayCreator::create(src->size(), dst->dtype(), c));
  tmp->copy_from(src);
  NBLA_HIP_CALL(nbla_hip_memcpy(dst->pointer<void>(), tmp->const_pointer<void>(),
                                (size_t)dst->size() * sizeof_dtype(dst->dtype()), 2, nullptr));
}

// Host -> device.
void synchronizer_cpu_array_hip_array(Array *src, Array *dst, int) {
  NBLA_CHECK(src->size() == dst->size(), error_code::unclassified, "Size mismatch.");
  hip_set_device(dst->context());
  if (src->size() == 0)
    return;
  if (src->dtype() == dst->dtype()) {
    NBLA_HIP_CALL(nbla_hip_memcpy(dst->pointer<void>(), src->const_pointer<void>(),
                                  (size_t)src->size() * sizeof_dtype(src->dtype()), 1, nullptr));
    return;
  }
  Context c = dst->context();
  c.array_class = "HipCachedArray";
  ArrayPtr tmp(ArrayCreator::create(src->size(), src->dtype(), c));
  NBLA_HIP_CALL(nbla_hip_memcpy(tmp->pointer<void>(), src->const_pointer<void>(),
                                (size_t)src->size() * sizeof_dtype(src->dtype()), 1, nullptr));
  dst->copy_from(tmp.get());
}

void synchronizer_hip_array_hip_array(Array *src, Array *dst, int) { dst->copy_from(src); }

// ------------------------------------------------------------------------- Hip
Hip::Hip()
    : naive_allocator_(make_shared<NaiveAllocator<HipMemory>>()),
      caching_allocator_(make_shared<CachingAllocatorWithBuckets<HipMemory>>()) {}
Hip::~Hip() {}
vector<string> Hip::array_classes() const { return array_classes_; }
void Hip::_set_array_classes(const vector<string> &a) { array_classes_ = a; }
void Hip::register_array_class(const string &name) { array_classes_.push_back(name); }
shared_ptr<Allocator> Hip::caching_allocator() { return caching_allocator_; }
shared_ptr<Allocator> Hip::naive_allocator() { return naive_allocator_; }
void Hip::free_unused_host_caches() {}
void Hip::device_synchronize(const string &device) {
  NBLA_HIP_CALL(nbla_hip_device_synchronize(hip_device_index(device)));
}
void Hip::default_stream_synchronize(const string &device) {
  NBLA_HIP_CALL(nbla_hip_set_device(hip_device_index(device)));
  NBLA_HIP_CALL(nbla_hip_stream_synchronize(nullptr));
}
void Hip::create_lms_streams(int) {}
int Hip::get_device_count() const {
  int n = 0;
  nbla_hip_get_device_count(&n);
  return n;
}

vector<string> hip_array_classes() { return SingletonManager::get<Hip>()->array_classes(); }
void hip_device_synchronize(const string &device) { SingletonManager::get<Hip>()->device_synchronize(device); }
int hip_get_device_count() { return SingletonManager::get<Hip>()->get_device_count(); }
vector<string> hip_get_devices() {
  vector<string> out;
  const int n = hip_get_device_count();
  for (int i = 0; i < n; ++i)
    out.push_back(std::to_string(i));
  return out;
}
void hip_clear_memory_cache() {
  SingletonManager::get<Hip>()->caching_allocator()->free_unused_caches();
  SingletonManager::get<Hip>()->naive_allocator()->free_unused_caches();
}

} // namespace nbla
