// Host arrays (mirrors include/nbla/array/cpu_array.hpp).
#ifndef NBLA_CPU_ARRAY_HPP_
#define NBLA_CPU_ARRAY_HPP_

#include <nbla/array.hpp>

namespace nbla {

// Host array backed by the naive (uncached) host allocator.
class NBLA_API CpuArray : public Array {
public:
  // Without `mem` the array takes its memory from the backend's allocator (cpu_array.cpp:25-31).
  CpuArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
           const Size_t offset = 0);
  virtual ~CpuArray();
  void copy_from(const Array *src_array) override;
  void zero() override;
  void fill(float value) override;
  static Context filter_context(const Context &ctx);
};

// Host array backed by the caching host allocator.
class NBLA_API CpuCachedArray : public CpuArray {
public:
  CpuCachedArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
                 const Size_t offset = 0);
  virtual ~CpuCachedArray();
  static Context filter_context(const Context &ctx);
};

// Plain host-to-host synchroniser (also the model for device synchronisers).
NBLA_API void synchronizer_cpu_array_cpu_array(Array *src, Array *dst, int async_flags = 0);
// Converting copy between two host buffers of any supported dtype pair.
NBLA_API void cpu_array_copy(const void *src, dtypes src_dtype, void *dst, dtypes dst_dtype, Size_t size);
NBLA_API void cpu_fill(void *dst, dtypes dtype, Size_t size, float value);

} // namespace nbla
#endif
