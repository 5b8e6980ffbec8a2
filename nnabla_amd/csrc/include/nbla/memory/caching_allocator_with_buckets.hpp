// Caching allocator with a small-block and a large-block pool per device
// (mirrors include/nbla/memory/caching_allocator_with_buckets.hpp:73-122 and
// src/nbla/memory/caching_allocator_with_buckets.cpp:107-215): requests are
// rounded to 512 B (below 1 MiB) or 128 KiB, small requests are carved from
// 1 MiB slabs, freed blocks merge with free neighbours and are kept for reuse.
#ifndef NBLA_CACHING_ALLOCATOR_WITH_BUCKETS_HPP_
#define NBLA_CACHING_ALLOCATOR_WITH_BUCKETS_HPP_

#include <nbla/memory/allocator.hpp>

#include <map>

namespace nbla {

class NBLA_API CachingAllocatorWithBucketsBase : public Allocator {
public:
  static constexpr size_t kRoundSmall = 512;
  static constexpr size_t kRoundLarge = 128 << 10;
  static constexpr size_t kSmallAllocSize = 1 << 20;
  typedef std::pair<size_t, Memory *> Key;
  typedef std::map<Key, shared_ptr<Memory>> CacheMap;
  typedef std::unordered_map<string, CacheMap> DeviceCacheMap;

  size_t round_size(size_t bytes) const;
  // Bytes sitting in the caches of a device (for tests and diagnostics).
  size_t get_cached_bytes(const string &device_id);

protected:
  DeviceCacheMap small_cache_, large_cache_;
  shared_ptr<Memory> alloc_impl(size_t bytes, const string &device_id) override;
  void free_impl(shared_ptr<Memory> memory) override;
  size_t free_unused_device_caches_impl(const string &device_id) override;
  vector<string> cached_devices() override;
  virtual shared_ptr<Memory> make_memory_impl(size_t bytes, const string &device_id) = 0;

private:
  void cache_insert(CacheMap &cache, shared_ptr<Memory> mem);
  size_t free_unused_in(CacheMap &cache, const string &device_id);
};

template <class MemoryType> class CachingAllocatorWithBuckets : public CachingAllocatorWithBucketsBase {
protected:
  shared_ptr<Memory> make_memory_impl(size_t bytes, const string &device_id) override {
    return make_shared<MemoryType>(bytes, device_id);
  }
};

} // namespace nbla
#endif
