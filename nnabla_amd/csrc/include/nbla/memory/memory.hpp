// A block of device (or host) memory that can be split and re-merged
// (mirrors include/nbla/memory/memory.hpp:74-347).
#ifndef NBLA_MEMORY_HPP_
#define NBLA_MEMORY_HPP_

#include <nbla/common.hpp>

namespace nbla {

class NBLA_API Memory {
  string device_id_;
  bool locked_ = false;
  Memory *next_ = nullptr;
  Memory *prev_ = nullptr;
  void disable() { ptr_ = nullptr; }

public:
  Memory(size_t bytes, const string &device_id);
  virtual ~Memory();
  Memory(const Memory &) = delete;
  Memory &operator=(const Memory &) = delete;

  size_t bytes() const { return bytes_; }
  string device_id() const { return device_id_; }
  void *pointer() { return ptr_; }
  const void *const_pointer() const { return ptr_; }
  bool locked() const { return locked_; }
  void lock() { locked_ = true; }
  void release() { locked_ = false; }
  Memory *prev() const { return prev_; }
  Memory *next() const { return next_; }
  // Neighbour blocks carved from the same allocation are held weakly through raw
  // pointers; the owning allocator keeps them alive.
  bool disabled() { return !ptr_; }

  // Obtains the memory from the device; throws error_code::memory on failure.
  void alloc();
  // Splits off [second_start, bytes) into a new block that becomes `next`.
  shared_ptr<Memory> divide(size_t second_start);
  // Absorbs an unlocked neighbour (which becomes disabled).
  void try_merge(Memory *from);
  static void associate_consecutive(Memory *left, Memory *right);

protected:
  size_t bytes_ = 0;
  void *ptr_ = nullptr;
  // Backend hooks.  An implementation keeps whatever owns the underlying allocation itself (CpuMemory and HipMemory
  // share one owner between all fragments carved from an allocation).
  virtual bool alloc_impl() = 0;
  virtual shared_ptr<Memory> divide_impl(size_t second_start) = 0;
  virtual void merge_next_impl(Memory *from) = 0;
  virtual void merge_prev_impl(Memory *from) = 0;
};

} // namespace nbla
#endif
