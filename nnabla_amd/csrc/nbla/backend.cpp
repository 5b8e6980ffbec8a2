// Backend registry, the host backend, and init_cpu().
#include <nbla/array/cpu_array.hpp>
#include <nbla/array_registry.hpp>
#include <nbla/backend_registry.hpp>
#include <nbla/cpu.hpp>
#include <nbla/init.hpp>
#include <nbla/memory/caching_allocator_with_buckets.hpp>
#include <nbla/memory/cpu_memory.hpp>
#include <nbla/memory/naive_allocator.hpp>

#include <mutex>

namespace nbla {

std::map<string, BackendUtils::BackendGetter> &BackendUtils::get_registry() {
  static std::map<string, BackendGetter> r;
  return r;
}
void BackendUtils::add_backend(const string &backend_name, BackendGetter backend_getter) {
  get_registry()[backend_name] = backend_getter;
}
BackendBase *BackendUtils::get_backend(const Context ctx) {
  init_cpu();
  NBLA_CHECK(!ctx.backend.empty(), error_code::unclassified, "Backend is empty.");
  const string first = ctx.backend[0];
  const string key = first.substr(0, first.find(':')); // "hip:float" -> "hip"
  auto it = get_registry().find(key);
  if (it == get_registry().end()) {
    vector<string> have;
    for (auto &kv : get_registry())
      have.push_back(kv.first);
    NBLA_ERROR(error_code::unclassified, "'%s' could not be found in [%s]", key.c_str(),
               string_join(have, ", ").c_str());
  }
  return it->second();
}
vector<string> BackendUtils::array_classes(const Context ctx) { return get_backend(ctx)->array_classes(); }
void BackendUtils::_set_array_classes(const Context ctx, const vector<string> &a) {
  get_backend(ctx)->_set_array_classes(a);
}
void BackendUtils::register_array_class(const Context ctx, const string &name) {
  get_backend(ctx)->register_array_class(name);
}
shared_ptr<Allocator> BackendUtils::caching_allocator(const Context ctx) { return get_backend(ctx)->caching_allocator(); }
shared_ptr<Allocator> BackendUtils::naive_allocator(const Context ctx) { return get_backend(ctx)->naive_allocator(); }
void BackendUtils::free_unused_host_caches(const Context ctx) { get_backend(ctx)->free_unused_host_caches(); }
void BackendUtils::device_synchronize(const Context ctx) { get_backend(ctx)->device_synchronize(ctx.device_id); }
void BackendUtils::default_stream_synchronize(const Context ctx) {
  get_backend(ctx)->default_stream_synchronize(ctx.device_id);
}
void BackendUtils::create_lms_streams(const Context ctx) { get_backend(ctx)->create_lms_streams(); }

// ------------------------------------------------------------------------- Cpu
Cpu::Cpu()
    : naive_allocator_(make_shared<NaiveAllocator<CpuMemory>>()),
      caching_allocator_(make_shared<CachingAllocatorWithBuckets<CpuMemory>>()) {}
Cpu::~Cpu() {}
vector<string> Cpu::array_classes() const { return array_classes_; }
void Cpu::_set_array_classes(const vector<string> &a) { array_classes_ = a; }
void Cpu::register_array_class(const string &name) { array_classes_.push_back(name); }
shared_ptr<Allocator> Cpu::caching_allocator() { return caching_allocator_; }
shared_ptr<Allocator> Cpu::naive_allocator() { return naive_allocator_; }
void Cpu::free_unused_host_caches() {
  caching_allocator_->free_unused_caches();
  naive_allocator_->free_unused_caches();
}
void Cpu::device_synchronize(const string &) {}
void Cpu::default_stream_synchronize(const string &) {}
void Cpu::create_lms_streams(int) {}

// -------------------------------------------------------------------- init_cpu
void init_cpu() {
  static std::mutex mtx;
  static bool done = false;
  std::lock_guard<std::mutex> lock(mtx);
  if (done)
    return;
  done = true;
  NBLA_REGISTER_BACKEND("cpu", []() { return SingletonManager::get<Cpu>(); });
  NBLA_REGISTER_ARRAY_CREATOR(CpuArray);
  SingletonManager::get<Cpu>()->register_array_class("CpuArray");
  NBLA_REGISTER_ARRAY_CREATOR(CpuCachedArray);
  SingletonManager::get<Cpu>()->register_array_class("CpuCachedArray");
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuArray, CpuCachedArray, synchronizer_cpu_array_cpu_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuCachedArray, CpuArray, synchronizer_cpu_array_cpu_array);
  NBLA_REGISTER_ARRAY_GROUP(CpuArray, CpuArray);
  NBLA_REGISTER_ARRAY_GROUP(CpuCachedArray, CpuArray);
  // No "cpu:float" Function implementations are registered: this build computes on the hip backend only.
}

void clear_all_singletons() { SingletonManager::clear(); }
vector<string> cpu_array_classes() { return SingletonManager::get<Cpu>()->array_classes(); }

} // namespace nbla
