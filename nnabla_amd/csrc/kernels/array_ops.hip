// Device memory management and the storage-level array operations (fill, dtype
// cast, ReLU) that the HipArray classes of the host layer are built on.
#include "common.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

constexpr int kBlk = 256;

unsigned grid_for(size_t size) {
  size_t b = (size + kBlk - 1) / kBlk;
  return (unsigned)(b > 16384 ? 16384 : (b < 1 ? 1 : b));
}

template <typename T> __global__ __launch_bounds__(kBlk) void fill_kernel(T *dst, size_t size, T value) {
  for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk)
    dst[i] = value;
}

template <typename Ta, typename Tb>
__global__ __launch_bounds__(kBlk) void cast_kernel(const Ta *__restrict__ src, Tb *__restrict__ dst, size_t size) {
  for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk)
    dst[i] = static_cast<Tb>(src[i]);
}

typedef float float4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(kBlk) void relu_kernel(const float *__restrict__ x, float *__restrict__ y, size_t n4,
                                                    size_t size, int vec) {
  if (vec) {
    for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < n4; i += (size_t)gridDim.x * kBlk) {
      float4_t v = reinterpret_cast<const float4_t *>(x)[i];
      // std::max(T(0), x): zero for negatives and for NaN-free -0.0 keeps +0.0
      v.x = v.x > 0.0f ? v.x : 0.0f;
      v.y = v.y > 0.0f ? v.y : 0.0f;
      v.z = v.z > 0.0f ? v.z : 0.0f;
      v.w = v.w > 0.0f ? v.w : 0.0f;
      reinterpret_cast<float4_t *>(y)[i] = v;
    }
    if (blockIdx.x == 0) {
      const size_t i = 4 * n4 + threadIdx.x;
      if (i < size)
        y[i] = x[i] > 0.0f ? x[i] : 0.0f;
    }
  } else {
    for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk)
      y[i] = x[i] > 0.0f ? x[i] : 0.0f;
  }
}

// y = x0 + x1, or dx (+)= dy when x1 is null (kAccum: dx already holds a gradient)
template <bool kSum, bool kAccum>
__global__ __launch_bounds__(kBlk) void add_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                   float *__restrict__ y, size_t n4, size_t size, int vec) {
  if (vec) {
    for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < n4; i += (size_t)gridDim.x * kBlk) {
      float4_t v = reinterpret_cast<const float4_t *>(a)[i];
      if (kSum)
        v += reinterpret_cast<const float4_t *>(b)[i];
      if (kAccum)
        v = reinterpret_cast<const float4_t *>(y)[i] + v;
      reinterpret_cast<float4_t *>(y)[i] = v;
    }
  }
  const size_t done = vec ? 4 * n4 : 0;
  for (size_t i = done + (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk) {
    float v = a[i];
    if (kSum)
      v += b[i];
    y[i] = kAccum ? y[i] + v : v;
  }
}

// Sub2, Mul2, Div2 on inputs of one shape (sub2.hpp:41, mul2.hpp:42, div2.hpp:44): y = op(x0, x1), and for the
// gradient of input kInput  dx = (accum ? dx : 0) + g(dy, x0, x1)  as base_transform_binary.hpp:286-336 forms it (the
// sum with the zeroed gradient included: it turns a -0 into +0).
enum { kOpSub2 = 0, kOpMul2 = 1, kOpDiv2 = 2 };
template <int kOp> __device__ __forceinline__ float binary2(float x0, float x1) {
  return kOp == kOpSub2 ? x0 - x1 : (kOp == kOpMul2 ? x0 * x1 : x0 / x1);
}
template <int kOp, int kInput> __device__ __forceinline__ float binary2_grad(float dy, float x0, float x1) {
  if (kOp == kOpSub2)
    return kInput == 0 ? dy : -dy;
  if (kOp == kOpMul2)
    return kInput == 0 ? dy * x1 : dy * x0;
  return kInput == 0 ? dy / x1 : -dy * x0 / (x1 * x1);
}
template <int kOp>
__global__ __launch_bounds__(kBlk) void binary2_kernel(const float *__restrict__ x0, const float *__restrict__ x1,
                                                       float *__restrict__ y, size_t n4, size_t size, int vec) {
  if (vec) {
    for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < n4; i += (size_t)gridDim.x * kBlk) {
      const float4_t a = reinterpret_cast<const float4_t *>(x0)[i], b = reinterpret_cast<const float4_t *>(x1)[i];
      float4_t v;
      v.x = binary2<kOp>(a.x, b.x), v.y = binary2<kOp>(a.y, b.y);
      v.z = binary2<kOp>(a.z, b.z), v.w = binary2<kOp>(a.w, b.w);
      reinterpret_cast<float4_t *>(y)[i] = v;
    }
  }
  const size_t done = vec ? 4 * n4 : 0;
  for (size_t i = done + (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk)
    y[i] = binary2<kOp>(x0[i], x1[i]);
}
// (dx may be the array dy lives in -- never one of x0 / x1 the other gradient still needs: no __restrict__ on dx)
template <int kOp, int kInput, bool kAccum>
__global__ __launch_bounds__(kBlk) void binary2_grad_kernel(const float *dy, const float *__restrict__ x0,
                                                            const float *__restrict__ x1, float *dx, size_t size) {
  for (size_t i = (size_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlk) {
    const float g = binary2_grad<kOp, kInput>(dy[i], kOp == kOpSub2 ? 0.0f : x0[i], kOp == kOpSub2 ? 0.0f : x1[i]);
    dx[i] = (kAccum ? dx[i] : 0.0f) + g;
  }
}
template <int kOp> int launch_binary2(const float *x0, const float *x1, float *y, size_t size, hipStream_t stream) {
  const int vec = aligned16(x0) && aligned16(x1) && aligned16(y);
  hipLaunchKernelGGL(binary2_kernel<kOp>, dim3(grid_for(vec ? size / 4 + 1 : size)), dim3(kBlk), 0, stream, x0, x1, y,
                     size / 4, size, vec);
  NBLA_HIP_LAUNCH_CHECK("binary2");
  return NBLA_HIP_OK;
}
template <int kOp, int kInput>
int launch_binary2_grad(const float *dy, const float *x0, const float *x1, float *dx, size_t size, int accum,
                        hipStream_t stream) {
  const dim3 g(grid_for(size)), b(kBlk);
  if (accum)
    hipLaunchKernelGGL((binary2_grad_kernel<kOp, kInput, true>), g, b, 0, stream, dy, x0, x1, dx, size);
  else
    hipLaunchKernelGGL((binary2_grad_kernel<kOp, kInput, false>), g, b, 0, stream, dy, x0, x1, dx, size);
  NBLA_HIP_LAUNCH_CHECK("binary2 backward");
  return NBLA_HIP_OK;
}

// dst[r * dst_stride + i] (+)= src[r * src_stride + i] for r < rows, i < len: the copies of Concatenate
template <bool kAccum>
__global__ __launch_bounds__(kBlk) void rows_copy_kernel(const float *__restrict__ src, int64_t src_stride,
                                                         float *__restrict__ dst, int64_t dst_stride, int64_t rows,
                                                         int64_t len) {
  const int64_t total = rows * len;
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < total; t += (int64_t)gridDim.x * kBlk) {
    const int64_t r = t / len, i = t - r * len;
    const float v = src[r * src_stride + i];
    float *d = dst + r * dst_stride + i;
    *d = kAccum ? *d + v : v;
  }
}

// nbla::dtypes codes (numpy compatible)
enum { DT_BOOL = 0, DT_BYTE, DT_UBYTE, DT_SHORT, DT_USHORT, DT_INT, DT_UINT, DT_LONG, DT_ULONG, DT_LONGLONG,
       DT_ULONGLONG, DT_FLOAT, DT_DOUBLE };

template <typename Ta> int cast_from(const void *src, void *dst, int dst_dtype, size_t size, hipStream_t s) {
  const Ta *p = static_cast<const Ta *>(src);
  const dim3 g(grid_for(size)), b(kBlk);
  switch (dst_dtype) {
  case DT_BOOL: hipLaunchKernelGGL((cast_kernel<Ta, bool>), g, b, 0, s, p, static_cast<bool *>(dst), size); break;
  case DT_BYTE: hipLaunchKernelGGL((cast_kernel<Ta, signed char>), g, b, 0, s, p, static_cast<signed char *>(dst), size); break;
  case DT_UBYTE: hipLaunchKernelGGL((cast_kernel<Ta, unsigned char>), g, b, 0, s, p, static_cast<unsigned char *>(dst), size); break;
  case DT_SHORT: hipLaunchKernelGGL((cast_kernel<Ta, short>), g, b, 0, s, p, static_cast<short *>(dst), size); break;
  case DT_USHORT: hipLaunchKernelGGL((cast_kernel<Ta, unsigned short>), g, b, 0, s, p, static_cast<unsigned short *>(dst), size); break;
  case DT_INT: hipLaunchKernelGGL((cast_kernel<Ta, int>), g, b, 0, s, p, static_cast<int *>(dst), size); break;
  case DT_UINT: hipLaunchKernelGGL((cast_kernel<Ta, unsigned int>), g, b, 0, s, p, static_cast<unsigned int *>(dst), size); break;
  case DT_LONG:
  case DT_LONGLONG: hipLaunchKernelGGL((cast_kernel<Ta, long long>), g, b, 0, s, p, static_cast<long long *>(dst), size); break;
  case DT_ULONG:
  case DT_ULONGLONG: hipLaunchKernelGGL((cast_kernel<Ta, unsigned long long>), g, b, 0, s, p, static_cast<unsigned long long *>(dst), size); break;
  case DT_FLOAT: hipLaunchKernelGGL((cast_kernel<Ta, float>), g, b, 0, s, p, static_cast<float *>(dst), size); break;
  case DT_DOUBLE: hipLaunchKernelGGL((cast_kernel<Ta, double>), g, b, 0, s, p, static_cast<double *>(dst), size); break;
  default: return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "unsupported destination dtype %d.", dst_dtype);
  }
  NBLA_HIP_LAUNCH_CHECK("cast");
  return NBLA_HIP_OK;
}

template <typename T> int fill_as(void *dst, size_t size, float value, hipStream_t s) {
  hipLaunchKernelGGL(fill_kernel<T>, dim3(grid_for(size)), dim3(kBlk), 0, s, static_cast<T *>(dst), size,
                     static_cast<T>(value));
  NBLA_HIP_LAUNCH_CHECK("fill");
  return NBLA_HIP_OK;
}

size_t dtype_bytes(int dtype) {
  switch (dtype) {
  case DT_BOOL: case DT_BYTE: case DT_UBYTE: return 1;
  case DT_SHORT: case DT_USHORT: return 2;
  case DT_INT: case DT_UINT: case DT_FLOAT: return 4;
  case DT_LONG: case DT_ULONG: case DT_LONGLONG: case DT_ULONGLONG: case DT_DOUBLE: return 8;
  }
  return 0;
}

} // namespace

int launch_clear_words(void *dst, size_t count, hipStream_t stream) {
  return fill_as<unsigned int>(dst, count, 0.0f, stream);
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_get_device_count(int *count) {
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    return fail_hip(e, "hipGetDeviceCount");
  }
  return NBLA_HIP_OK;
}

int nbla_hip_set_device(int device) {
  hipError_t e = hipSetDevice(device);
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipSetDevice");
}

int nbla_hip_malloc(void **ptr, size_t bytes, int device) {
  hipError_t e = hipSetDevice(device);
  if (e == hipSuccess)
    e = hipMalloc(ptr, bytes ? bytes : 1);
  if (e != hipSuccess) {
    *ptr = nullptr;
    (void)hipGetLastError(); // a failed allocation must not poison the next call
    return fail_hip(e, "hipMalloc");
  }
  return NBLA_HIP_OK;
}

int nbla_hip_free(void *ptr, int device) {
  if (!ptr)
    return NBLA_HIP_OK;
  hipError_t e = hipSetDevice(device);
  if (e == hipSuccess)
    e = hipFree(ptr);
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipFree");
}

int nbla_hip_mem_info(int device, size_t *free_bytes, size_t *total_bytes) {
  hipError_t e = hipSetDevice(device);
  if (e == hipSuccess)
    e = hipMemGetInfo(free_bytes, total_bytes);
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipMemGetInfo");
}

int nbla_hip_memcpy(void *dst, const void *src, size_t bytes, int kind, void *stream) {
  if (bytes == 0)
    return NBLA_HIP_OK;
  hipMemcpyKind k;
  switch (kind) {
  case 1: k = hipMemcpyHostToDevice; break;
  case 2: k = hipMemcpyDeviceToHost; break;
  case 3: k = hipMemcpyDeviceToDevice; break;
  default: return fail(NBLA_HIP_ERR_VALUE, "invalid memcpy kind %d.", kind);
  }
  hipError_t e = hipMemcpyAsync(dst, src, bytes, k, as_stream(stream));
  if (e == hipSuccess && k != hipMemcpyDeviceToDevice)
    e = hipStreamSynchronize(as_stream(stream)); // host buffers are pageable: complete before returning
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipMemcpyAsync");
}

int nbla_hip_device_synchronize(int device) {
  hipError_t e = hipSetDevice(device);
  if (e == hipSuccess)
    e = hipDeviceSynchronize();
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipDeviceSynchronize");
}

int nbla_hip_stream_synchronize(void *stream) {
  hipError_t e = hipStreamSynchronize(as_stream(stream));
  return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipStreamSynchronize");
}

int nbla_hip_fill(void *dst, int dtype, size_t size, float value, void *stream_) {
  if (size == 0)
    return NBLA_HIP_OK;
  hipStream_t s = as_stream(stream_);
  if (value == 0.0f) { // all-zero bytes for every dtype
    const size_t bytes = size * dtype_bytes(dtype);
    if (bytes % 4 == 0)
      return fill_as<unsigned int>(dst, bytes / 4, 0.0f, s);
    return fill_as<unsigned char>(dst, bytes, 0.0f, s);
  }
  switch (dtype) {
  case DT_BOOL: return fill_as<bool>(dst, size, value, s);
  case DT_BYTE: return fill_as<signed char>(dst, size, value, s);
  case DT_UBYTE: return fill_as<unsigned char>(dst, size, value, s);
  case DT_SHORT: return fill_as<short>(dst, size, value, s);
  case DT_USHORT: return fill_as<unsigned short>(dst, size, value, s);
  case DT_INT: return fill_as<int>(dst, size, value, s);
  case DT_UINT: return fill_as<unsigned int>(dst, size, value, s);
  case DT_LONG: case DT_LONGLONG: return fill_as<long long>(dst, size, value, s);
  case DT_ULONG: case DT_ULONGLONG: return fill_as<unsigned long long>(dst, size, value, s);
  case DT_FLOAT: return fill_as<float>(dst, size, value, s);
  case DT_DOUBLE: return fill_as<double>(dst, size, value, s);
  }
  return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "unsupported dtype %d.", dtype);
}

int nbla_hip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t size, void *stream_) {
  if (size == 0)
    return NBLA_HIP_OK;
  hipStream_t s = as_stream(stream_);
  const bool same = src_dtype == dst_dtype ||
                    ((src_dtype == DT_LONG || src_dtype == DT_LONGLONG) && (dst_dtype == DT_LONG || dst_dtype == DT_LONGLONG)) ||
                    ((src_dtype == DT_ULONG || src_dtype == DT_ULONGLONG) && (dst_dtype == DT_ULONG || dst_dtype == DT_ULONGLONG));
  if (same) {
    hipError_t e = hipMemcpyAsync(dst, src, size * dtype_bytes(src_dtype), hipMemcpyDeviceToDevice, s);
    return e == hipSuccess ? NBLA_HIP_OK : fail_hip(e, "hipMemcpyAsync");
  }
  switch (src_dtype) {
  case DT_BOOL: return cast_from<bool>(src, dst, dst_dtype, size, s);
  case DT_BYTE: return cast_from<signed char>(src, dst, dst_dtype, size, s);
  case DT_UBYTE: return cast_from<unsigned char>(src, dst, dst_dtype, size, s);
  case DT_SHORT: return cast_from<short>(src, dst, dst_dtype, size, s);
  case DT_USHORT: return cast_from<unsigned short>(src, dst, dst_dtype, size, s);
  case DT_INT: return cast_from<int>(src, dst, dst_dtype, size, s);
  case DT_UINT: return cast_from<unsigned int>(src, dst, dst_dtype, size, s);
  case DT_LONG: case DT_LONGLONG: return cast_from<long long>(src, dst, dst_dtype, size, s);
  case DT_ULONG: case DT_ULONGLONG: return cast_from<unsigned long long>(src, dst, dst_dtype, size, s);
  case DT_FLOAT: return cast_from<float>(src, dst, dst_dtype, size, s);
  case DT_DOUBLE: return cast_from<double>(src, dst, dst_dtype, size, s);
  }
  return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "unsupported source dtype %d.", src_dtype);
}

int nbla_hip_add2_f32(const float *x0, const float *x1, float *y, size_t size, void *stream) {
  if (size == 0)
    return NBLA_HIP_OK;
  const int vec = aligned16(x0) && aligned16(x1) && aligned16(y);
  hipLaunchKernelGGL((add_kernel<true, false>), dim3(grid_for(vec ? size / 4 + 1 : size)), dim3(kBlk), 0,
                     as_stream(stream), x0, x1, y, size / 4, size, vec);
  NBLA_HIP_LAUNCH_CHECK("add2");
  return NBLA_HIP_OK;
}

int nbla_hip_add2_backward_f32(const float *dy, float *dx, size_t size, int accum, void *stream) {
  if (size == 0 || (dx == dy && !accum))
    return NBLA_HIP_OK;
  const int vec = aligned16(dy) && aligned16(dx);
  const dim3 g(grid_for(vec ? size / 4 + 1 : size)), b(kBlk);
  if (accum)
    hipLaunchKernelGGL((add_kernel<false, true>), g, b, 0, as_stream(stream), dy, nullptr, dx, size / 4, size, vec);
  else
    hipLaunchKernelGGL((add_kernel<false, false>), g, b, 0, as_stream(stream), dy, nullptr, dx, size / 4, size, vec);
  NBLA_HIP_LAUNCH_CHECK("add2 backward");
  return NBLA_HIP_OK;
}

int nbla_hip_binary2_f32(int op, const float *x0, const float *x1, float *y, size_t size, void *stream) {
  if (size == 0)
    return NBLA_HIP_OK;
  switch (op) {
  case kOpSub2: return launch_binary2<kOpSub2>(x0, x1, y, size, as_stream(stream));
  case kOpMul2: return launch_binary2<kOpMul2>(x0, x1, y, size, as_stream(stream));
  case kOpDiv2: return launch_binary2<kOpDiv2>(x0, x1, y, size, as_stream(stream));
  }
  return fail(NBLA_HIP_ERR_VALUE, "binary2: unknown operation %d.", op);
}

int nbla_hip_binary2_backward_f32(int op, int input, const float *dy, const float *x0, const float *x1, float *dx,
                                  size_t size, int accum, void *stream) {
  if (size == 0)
    return NBLA_HIP_OK;
  if (input != 0 && input != 1)
    return fail(NBLA_HIP_ERR_VALUE, "binary2 backward: input %d is not 0 or 1.", input);
  hipStream_t s = as_stream(stream);
#define NBLA_BINARY2_GRAD(OP)                                                                                          \
  return input == 0 ? launch_binary2_grad<OP, 0>(dy, x0, x1, dx, size, accum, s)                                       \
                    : launch_binary2_grad<OP, 1>(dy, x0, x1, dx, size, accum, s)
  switch (op) {
  case kOpSub2: NBLA_BINARY2_GRAD(kOpSub2);
  case kOpMul2: NBLA_BINARY2_GRAD(kOpMul2);
  case kOpDiv2: NBLA_BINARY2_GRAD(kOpDiv2);
  }
#undef NBLA_BINARY2_GRAD
  return fail(NBLA_HIP_ERR_VALUE, "binary2 backward: unknown operation %d.", op);
}

int nbla_hip_copy_rows_f32(const float *src, int64_t src_stride, float *dst, int64_t dst_stride, int64_t rows,
                           int64_t len, int accum, void *stream) {
  if (rows < 0 || len < 0 || src_stride < len || dst_stride < len)
    return fail(NBLA_HIP_ERR_VALUE, "copy_rows: invalid sizes (rows=%lld, len=%lld, strides %lld / %lld).",
                (long long)rows, (long long)len, (long long)src_stride, (long long)dst_stride);
  if (rows == 0 || len == 0)
    return NBLA_HIP_OK;
  const dim3 g(grid_for((size_t)(rows * len))), b(kBlk);
  if (accum)
    hipLaunchKernelGGL(rows_copy_kernel<true>, g, b, 0, as_stream(stream), src, src_stride, dst, dst_stride, rows, len);
  else
    hipLaunchKernelGGL(rows_copy_kernel<false>, g, b, 0, as_stream(stream), src, src_stride, dst, dst_stride, rows, len);
  NBLA_HIP_LAUNCH_CHECK("copy_rows");
  return NBLA_HIP_OK;
}

int nbla_hip_relu_f32(const float *x, float *y, size_t size, void *stream) {
  if (size == 0)
    return NBLA_HIP_OK;
  const int vec = aligned16(x) && aligned16(y);
  hipLaunchKernelGGL(relu_kernel, dim3(grid_for(vec ? size / 4 + 1 : size)), dim3(kBlk), 0, as_stream(stream), x, y,
                     size / 4, size, vec);
  NBLA_HIP_LAUNCH_CHECK("relu");
  return NBLA_HIP_OK;
}

} // extern "C"
