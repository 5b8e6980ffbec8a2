// Device arrays of the hip backend and their synchronisers with the host array classes
// (the counterparts of include/nbla/array/cpu_array.hpp).
#ifndef NBLA_HIP_ARRAY_HPP_
#define NBLA_HIP_ARRAY_HPP_

#include <nbla/array.hpp>

namespace nbla {

// Device array backed by the naive (uncached) device allocator.
class NBLA_API HipArray : public Array {
protected:
  int device_;

public:
  // Without `mem` the array takes its memory from the hip backend's allocator, as CpuArray does from the host's.
  HipArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
           const Size_t offset = 0);
  virtual ~HipArray();
  void copy_from(const Array *src_array) override;
  void zero() override;
  void fill(float value) override;
  static Context filter_context(const Context &ctx);
};

// Device array backed by the caching device allocator (the default array class of the hip context).
class NBLA_API HipCachedArray : public HipArray {
public:
  HipCachedArray(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
                 const Size_t offset = 0);
  virtual ~HipCachedArray();
  static Context filter_context(const Context &ctx);
};

// Host <-> device transfers; a dtype change is done on the device side of the transfer.
NBLA_API void synchronizer_hip_array_cpu_array(Array *src, Array *dst, int async_flags = 0);
NBLA_API void synchronizer_cpu_array_hip_array(Array *src, Array *dst, int async_flags = 0);
NBLA_API void synchronizer_hip_array_hip_array(Array *src, Array *dst, int async_flags = 0);

} // namespace nbla
#endif
