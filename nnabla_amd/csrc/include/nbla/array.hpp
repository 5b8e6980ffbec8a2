// One typed buffer on one device (mirrors include/nbla/array.hpp).
#ifndef NBLA_ARRAY_HPP_
#define NBLA_ARRAY_HPP_

#include <nbla/context.hpp>
#include <nbla/exception.hpp>
#include <nbla/memory/allocator.hpp>

namespace nbla {

class NBLA_API Array {
protected:
  Size_t size_;
  dtypes dtype_;
  Context ctx_;
  AllocatorMemoryPtr mem_;
  Size_t offset_; // elements into mem_ (narrowed views)

public:
  Array(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
        const Size_t offset = 0);
  virtual ~Array();
  Array(const Array &) = delete;
  Array &operator=(const Array &) = delete;

  template <typename T = void> T *pointer() {
    return reinterpret_cast<T *>(static_cast<char *>(mem_->pointer()) + offset_ * sizeof_dtype(dtype_));
  }
  template <typename T = void> const T *const_pointer() const {
    return reinterpret_cast<const T *>(static_cast<const char *>(mem_->const_pointer()) +
                                       offset_ * sizeof_dtype(dtype_));
  }
  dtypes dtype() const { return dtype_; }
  Size_t size() const { return size_; }
  Size_t offset() const { return offset_; }
  const Context &context() const { return ctx_; }
  AllocatorMemoryPtr memory() const { return mem_; }

  // Element-wise copy with dtype conversion from an array of the same class family.
  virtual void copy_from(const Array *src_array) = 0;
  virtual void zero() = 0;
  virtual void fill(float value) = 0;
  // Blocks until pending asynchronous work on this array has finished.
  virtual void wait_event(const Context &ctx, int async_flags = 0);

  static Size_t size_as_bytes(Size_t size, dtypes dtype) { return size * (Size_t)sizeof_dtype(dtype); }
};
typedef shared_ptr<Array> ArrayPtr;
typedef shared_ptr<const Array> ConstArrayPtr;

} // namespace nbla
#endif
