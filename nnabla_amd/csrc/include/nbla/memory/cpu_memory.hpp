// Host memory block (mirrors include/nbla/memory/cpu_memory.hpp, src/nbla/memory/cpu_memory.cpp:31-80).
#ifndef NBLA_CPU_MEMORY_HPP_
#define NBLA_CPU_MEMORY_HPP_

#include <nbla/memory/memory.hpp>

namespace nbla {

class NBLA_API CpuMemory : public Memory {
public:
  CpuMemory(size_t bytes, const string &device_id);
  ~CpuMemory();

protected:
  // Owner of the allocation this block was carved from; shared by all of its fragments, so the allocation is
  // returned when the last fragment goes away, in whatever order that happens.
  shared_ptr<void> root_;
  CpuMemory(size_t bytes, const string &device_id, void *ptr);
  bool alloc_impl() override;
  shared_ptr<Memory> divide_impl(size_t second_start) override;
  void merge_next_impl(Memory *from) override;
  void merge_prev_impl(Memory *from) override;
};

} // namespace nbla
#endif
