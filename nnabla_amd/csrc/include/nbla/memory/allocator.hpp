// Allocator interface and the RAII handle arrays hold
// (mirrors include/nbla/memory/allocator.hpp:41-265).
#ifndef NBLA_ALLOCATOR_HPP_
#define NBLA_ALLOCATOR_HPP_

#include <nbla/memory/memory.hpp>

#include <functional>
#include <mutex>
#include <unordered_map>

namespace nbla {

class Allocator;

// Owns one Memory block on behalf of an Array; returns it to its allocator when destroyed.
class NBLA_API AllocatorMemory {
  shared_ptr<Memory> memory_;
  shared_ptr<Allocator> allocator_;

public:
  AllocatorMemory();
  AllocatorMemory(shared_ptr<Memory> memory, shared_ptr<Allocator> allocator);
  ~AllocatorMemory();
  AllocatorMemory(AllocatorMemory &&rhs);
  AllocatorMemory &operator=(AllocatorMemory &&rhs);
  AllocatorMemory(const AllocatorMemory &) = delete;
  AllocatorMemory &operator=(const AllocatorMemory &) = delete;
  shared_ptr<Memory> memory() { return memory_; }
  size_t bytes() const { return memory_ ? memory_->bytes() : 0; }
  string device_id() const { return memory_->device_id(); }
  void *pointer() { return memory_ ? memory_->pointer() : nullptr; }
  const void *const_pointer() const { return memory_ ? memory_->const_pointer() : nullptr; }

private:
  void release();
};
typedef shared_ptr<AllocatorMemory> AllocatorMemoryPtr;

class NBLA_API Allocator : public std::enable_shared_from_this<Allocator> {
public:
  Allocator() {}
  virtual ~Allocator() {}
  // Requests at least `bytes` on `device_id` (zero-byte requests get the minimum block).
  AllocatorMemoryPtr alloc(size_t bytes, const string &device_id);
  // Called by AllocatorMemory's destructor.
  void free(shared_ptr<Memory> memory);
  // Releases cached, currently unused blocks back to the device; returns the bytes freed.
  size_t free_unused_caches();
  size_t free_unused_device_caches(const string &device_id);
  // Bytes handed out by the device and still held (in use or cached), per device.
  size_t get_total_allocated_bytes(const string &device_id);

protected:
  std::mutex mutex_;
  std::unordered_map<string, size_t> device_bytes_;
  // Tries mem->alloc(); on error_code::memory frees this device's unused caches and retries once.
  void alloc_retry(shared_ptr<Memory> mem);
  virtual shared_ptr<Memory> alloc_impl(size_t bytes, const string &device_id) = 0;
  virtual void free_impl(shared_ptr<Memory> memory) = 0;
  virtual size_t free_unused_device_caches_impl(const string &device_id) = 0;
  virtual vector<string> cached_devices() = 0;
  void note_device_alloc(const string &device_id, size_t bytes) { device_bytes_[device_id] += bytes; }
  void note_device_free(const string &device_id, size_t bytes) { device_bytes_[device_id] -= bytes; }
};

} // namespace nbla
#endif
