// Shared host/device helpers of the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include "nbla_hip_kernels.h"

namespace nbla_hip {

// Records a message for nbla_hip_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);
int fail_hip(hipError_t err, const char *what);

// Makes sure the current device has been initialised (tables uploaded).
int ensure_init();

// Resolves, once per device and with that device current, the address of the fixed scratch array behind
// nbla_hip_min_max_quantize_static_f32 (defined beside that array).  Called by nbla_hip_init.
int register_static_scratch(int device);

// Number of binades a positive finite fp32 value can fall into: 23 subnormal
// binades (leading bit 0..22) followed by exponent fields 1..254.
constexpr int kNumBinades = 277;
enum CutTable { kCutPow2Round = 0, kCutInqExponent = 1, kCutInqN1 = 2, kNumCutTables = 3 };

// Device address of cut table `which` on the current device.
const uint32_t *device_cut_table(int which);

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Raises a kernel's dynamic LDS limit on the current device, once per device (`done` holds one bit per device; the
// attribute belongs to the device that is current when it is set).
inline int allow_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done, const char *what) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail_hip(e, "hipGetDevice");
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit)
    return NBLA_HIP_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess)
    return fail_hip(e, what);
  done.fetch_or(bit, std::memory_order_release);
  return NBLA_HIP_OK;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned256(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 255u) == 0; }

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define NBLA_HIP_LAUNCH_CHECK(what)                                                                                    \
  do {                                                                                                                 \
    hipError_t e__ = hipGetLastError();                                                                                \
    if (e__ != hipSuccess)                                                                                             \
      return ::nbla_hip::fail_hip(e__, what);                                                                          \
  } while (0)

// ---------------------------------------------------------------- device side

// Binade index of a non-zero, finite |x| given as its bit pattern.
__device__ __forceinline__ int binade_of(uint32_t u) {
  const uint32_t e = u >> 23;
  return e ? (int)e + 22 : 31 - __clz((int)u);
}
// Unbiased exponent E (value in [2^E, 2^(E+1))) of binade `idx`.
__device__ __forceinline__ int binade_exponent(int idx) { return idx - 149; }

// 2^e as fp32 for e in [-149, 127].
__device__ __forceinline__ float pow2_int(int e) {
  const uint32_t bits = (e >= -126) ? ((uint32_t)(e + 127) << 23) : (1u << (e + 149));
  return __uint_as_float(bits);
}

// roundf: to nearest, halves away from zero (std::round on fp32).
__device__ __forceinline__ float round_half_away(float t) {
  const float r = truncf(t);
  const float d = fabsf(t - r); // exact
  return (d >= 0.5f) ? r + copysignf(1.0f, t) : r;
}

} // namespace nbla_hip
