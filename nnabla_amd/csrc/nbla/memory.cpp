// Memory blocks, allocators and host memory.
#include <nbla/exception.hpp>
#include <nbla/memory/caching_allocator_with_buckets.hpp>
#include <nbla/memory/cpu_memory.hpp>

#include <cstdlib>

namespace nbla {

// ---------------------------------------------------------------------- Memory
Memory::Memory(size_t bytes, const string &device_id) : device_id_(device_id), bytes_(bytes) {}

Memory::~Memory() {
  // Unlink from the chain of blocks carved from the same allocation.
  if (prev_)
    prev_->next_ = next_;
  if (next_)
    next_->prev_ = prev_;
}

void Memory::alloc() {
  NBLA_CHECK(!ptr_, error_code::value, "Allocation called twice.");
  NBLA_CHECK(alloc_impl(), error_code::memory, "%s allocation failed. (%zu bytes on device %s)",
             "Memory", bytes_, device_id_.c_str());
}

void Memory::associate_consecutive(Memory *left, Memory *right) {
  if (left)
    left->next_ = right;
  if (right)
    right->prev_ = left;
}

shared_ptr<Memory> Memory::divide(size_t second_start) {
  NBLA_CHECK(second_start > 0 && second_start < bytes_, error_code::value,
             "`second_start` must be in (0, %zu). Given %zu.", bytes_, second_start);
  shared_ptr<Memory> second = divide_impl(second_start);
  bytes_ = second_start;
  associate_consecutive(second.get(), next_);
  associate_consecutive(this, second.get());
  return second;
}

void Memory::try_merge(Memory *from) {
  if (!from || from->locked() || from->disabled())
    return;
  if (from == next_) {
    merge_next_impl(from);
    bytes_ += from->bytes_;
    associate_consecutive(this, from->next_);
  } else if (from == prev_) {
    merge_prev_impl(from);
    bytes_ += from->bytes_;
    associate_consecutive(from->prev_, this);
  } else {
    return;
  }
  from->prev_ = from->next_ = nullptr;
  from->disable();
}

// ------------------------------------------------------------- AllocatorMemory
AllocatorMemory::AllocatorMemory() {}
AllocatorMemory::AllocatorMemory(shared_ptr<Memory> memory, shared_ptr<Allocator> allocator)
    : memory_(memory), allocator_(allocator) {}
void AllocatorMemory::release() {
  if (memory_ && allocator_)
    allocator_->free(memory_);
  memory_.reset();
  allocator_.reset();
}
AllocatorMemory::~AllocatorMemory() { release(); }
AllocatorMemory::AllocatorMemory(AllocatorMemory &&rhs) { *this = std::move(rhs); }
AllocatorMemory &AllocatorMemory::operator=(AllocatorMemory &&rhs) {
  if (this != &rhs) {
    release();
    memory_ = std::move(rhs.memory_);
    allocator_ = std::move(rhs.allocator_);
  }
  return *this;
}

// ------------------------------------------------------------------- Allocator
AllocatorMemoryPtr Allocator::alloc(size_t bytes, const string &device_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  shared_ptr<Memory> mem = alloc_impl(bytes, device_id);
  mem->lock();
  return make_shared<AllocatorMemory>(mem, shared_from_this());
}

void Allocator::free(shared_ptr<Memory> memory) {
  std::lock_guard<std::mutex> lock(mutex_);
  memory->release();
  free_impl(memory);
}

size_t Allocator::free_unused_caches() {
  std::lock_guard<std::mutex> lock(mutex_);
  size_t freed = 0;
  for (const string &dev : cached_devices())
    freed += free_unused_device_caches_impl(dev);
  return freed;
}

size_t Allocator::free_unused_device_caches(const string &device_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  return free_unused_device_caches_impl(device_id);
}

size_t Allocator::get_total_allocated_bytes(const string &device_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = device_bytes_.find(device_id);
  return it == device_bytes_.end() ? 0 : it->second;
}

void Allocator::alloc_retry(shared_ptr<Memory> mem) {
  try {
    mem->alloc();
  } catch (const Exception &e) {
    if (e.code() != error_code::memory)
      throw;
    free_unused_device_caches_impl(mem->device_id()); // give cached blocks back and try once more
    mem->alloc();
  }
}

// --------------------------------------------- CachingAllocatorWithBucketsBase
size_t CachingAllocatorWithBucketsBase::round_size(size_t bytes) const {
  if (bytes < kRoundSmall)
    return kRoundSmall;
  const size_t unit = bytes < kSmallAllocSize ? kRoundSmall : kRoundLarge;
  return (bytes + unit - 1) / unit * unit;
}

void CachingAllocatorWithBucketsBase::cache_insert(CacheMap &cache, shared_ptr<Memory> mem) {
  cache[Key{mem->bytes(), mem.get()}] = mem;
}

shared_ptr<Memory> CachingAllocatorWithBucketsBase::alloc_impl(size_t orig_bytes, const string &device_id) {
  const size_t bytes = round_size(orig_bytes);
  const bool small = bytes <= kSmallAllocSize;
  CacheMap &cache = small ? small_cache_[device_id] : large_cache_[device_id];
  shared_ptr<Memory> mem;
  auto it = cache.lower_bound(Key{bytes, nullptr});
  if (it != cache.end()) {
    mem = it->second;
    cache.erase(it);
  } else {
    const size_t alloc_bytes = small ? kSmallAllocSize : bytes;
    mem = make_memory_impl(alloc_bytes, device_id);
    alloc_retry(mem);
    note_device_alloc(device_id, alloc_bytes);
  }
  // Split off what is not needed when the remainder is worth keeping.
  const size_t remainder = mem->bytes() - bytes;
  if (small ? remainder >= kRoundSmall : remainder > kSmallAllocSize) {
    shared_ptr<Memory> rest = mem->divide(bytes);
    cache_insert(cache, rest);
  }
  return mem;
}

void CachingAllocatorWithBucketsBase::free_impl(shared_ptr<Memory> memory) {
  const string dev = memory->device_id();
  // Large-pool blocks and their fragments are always above 1 MiB, small-pool ones never are.
  const bool small = memory->bytes() <= kSmallAllocSize;
  CacheMap &cache = small ? small_cache_[dev] : large_cache_[dev];
  // Merge with free neighbours (they sit in the same cache).
  for (Memory *nb : {memory->next(), memory->prev()}) {
    if (!nb || nb->locked() || nb->disabled())
      continue;
    auto it = cache.find(Key{nb->bytes(), nb});
    if (it == cache.end())
      continue; // belongs to the other pool: never merged across pools
    shared_ptr<Memory> keep = it->second; // alive until the merge has read it
    cache.erase(it);
    memory->try_merge(nb);
  }
  cache_insert(cache, memory);
}

size_t CachingAllocatorWithBucketsBase::free_unused_in(CacheMap &cache, const string &device_id) {
  size_t freed = 0;
  for (auto it = cache.begin(); it != cache.end();) {
    Memory *m = it->second.get();
    if (!m->prev() && !m->next()) { // a whole allocation, not a fragment
      freed += m->bytes();
      note_device_free(device_id, m->bytes());
      it = cache.erase(it);
    } else {
      ++it;
    }
  }
  return freed;
}

size_t CachingAllocatorWithBucketsBase::free_unused_device_caches_impl(const string &device_id) {
  size_t freed = 0;
  if (small_cache_.count(device_id))
    freed += free_unused_in(small_cache_[device_id], device_id);
  if (large_cache_.count(device_id))
    freed += free_unused_in(large_cache_[device_id], device_id);
  return freed;
}

vector<string> CachingAllocatorWithBucketsBase::cached_devices() {
  vector<string> devs;
  for (auto &kv : small_cache_)
    devs.push_back(kv.first);
  for (auto &kv : large_cache_)
    if (!small_cache_.count(kv.first))
      devs.push_back(kv.first);
  return devs;
}

size_t CachingAllocatorWithBucketsBase::get_cached_bytes(const string &device_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  size_t total = 0;
  for (auto *pool : {&small_cache_, &large_cache_})
    if (pool->count(device_id))
      for (auto &kv : (*pool)[device_id])
        total += kv.second->bytes();
  return total;
}

// ------------------------------------------------------------------- CpuMemory
CpuMemory::CpuMemory(size_t bytes, const string &device_id) : Memory(bytes, device_id) {}
CpuMemory::CpuMemory(size_t bytes, const string &device_id, void *ptr) : Memory(bytes, device_id) { ptr_ = ptr; }
CpuMemory::~CpuMemory() {}
bool CpuMemory::alloc_impl() {
  void *p = nullptr;
  if (::posix_memalign(&p, 64, bytes_ ? bytes_ : 1) != 0)
    return false;
  ptr_ = p;
  root_ = shared_ptr<void>(p, [](void *q) { ::free(q); });
  return true;
}
shared_ptr<Memory> CpuMemory::divide_impl(size_t second_start) {
  CpuMemory *second = new CpuMemory(bytes_ - second_start, device_id(), static_cast<char *>(ptr_) + second_start);
  second->root_ = root_;
  return shared_ptr<Memory>(second);
}
void CpuMemory::merge_next_impl(Memory *) {}
void CpuMemory::merge_prev_impl(Memory *from) { ptr_ = from->pointer(); }

} // namespace nbla
