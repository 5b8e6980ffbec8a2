// A block of device memory obtained with hipMalloc (through the C-ABI), splittable by pointer offset
// (the counterpart of include/nbla/memory/cpu_memory.hpp).
#ifndef NBLA_HIP_MEMORY_HPP_
#define NBLA_HIP_MEMORY_HPP_

#include <nbla/exception.hpp>
#include <nbla/memory/memory.hpp>

namespace nbla {

class NBLA_API HipMemory : public Memory {
public:
  HipMemory(size_t bytes, const string &device_id);
  ~HipMemory();

protected:
  // Owner of the hipMalloc'ed block this memory was carved from; every fragment shares it, so the block goes back
  // to the device when the last fragment is destroyed, in whatever order the allocator drops them.
  shared_ptr<void> root_;
  HipMemory(size_t bytes, const string &device_id, void *ptr);
  bool alloc_impl() override;
  shared_ptr<Memory> divide_impl(size_t second_start) override;
  void merge_next_impl(Memory *from) override;
  void merge_prev_impl(Memory *from) override;
};

} // namespace nbla
#endif
