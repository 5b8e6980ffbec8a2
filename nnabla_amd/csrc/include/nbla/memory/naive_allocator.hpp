// Allocator without caching: every request goes to the device
// (mirrors include/nbla/memory/naive_allocator.hpp:34-60).
#ifndef NBLA_NAIVE_ALLOCATOR_HPP_
#define NBLA_NAIVE_ALLOCATOR_HPP_

#include <nbla/memory/allocator.hpp>

namespace nbla {

template <class MemoryType> class NaiveAllocator : public Allocator {
protected:
  shared_ptr<Memory> alloc_impl(size_t bytes, const string &device_id) override {
    auto mem = make_shared<MemoryType>(bytes ? bytes : 1, device_id);
    this->alloc_retry(mem);
    this->note_device_alloc(device_id, mem->bytes());
    return mem;
  }
  void free_impl(shared_ptr<Memory> memory) override { this->note_device_free(memory->device_id(), memory->bytes()); }
  size_t free_unused_device_caches_impl(const string &) override { return 0; }
  vector<string> cached_devices() override { return {}; }
};

} // namespace nbla
#endif
