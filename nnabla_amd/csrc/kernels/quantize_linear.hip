// QuantizeLinear, DequantizeLinear (broadcast scale / zero point, each arithmetic step rounded on its own as the
// reference's chain of Div2 / round / Add2 / saturate does) and Prune (k-th smallest |x| by a three-pass radix
// select over the magnitude bits, then a masked copy).  All HBM-bound; 128-bit accesses where the layout allows.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "quantize_common.hpp"

#include <cmath>

namespace nbla_hip {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxDims = 6;

// x viewed as up to kMaxDims dense dimensions (innermost last); a parameter's stride is 0 where it broadcasts.
struct Broadcast {
  int nd;
  int64_t size[kMaxDims], sstride[kMaxDims], zstride[kMaxDims];
};

// Merge neighbouring dimensions in which both parameters behave alike (both broadcast, or both dense and
// contiguous with the neighbour).  Returns false when more than kMaxDims remain.
bool make_broadcast(Broadcast &b, const int64_t *xshape, const int64_t *sshape, const int64_t *zshape, int ndim) {
  int64_t size[32], sb[32], zb[32];
  int n = 0;
  for (int i = 0; i < ndim; ++i) {
    if (xshape[i] == 1)
      continue;
    const int64_t s = sshape[i] != 1, z = zshape[i] != 1;
    if (n && sb[n - 1] == s && zb[n - 1] == z)
      size[n - 1] *= xshape[i];
    else {
      if (n == 32)
        return false;
      size[n] = xshape[i], sb[n] = s, zb[n] = z, ++n;
    }
  }
  if (n == 0)
    size[0] = 1, sb[0] = zb[0] = 0, n = 1;
  if (n > kMaxDims)
    return false;
  b.nd = n;
  int64_t ss = 1, zs = 1;
  for (int i = n - 1; i >= 0; --i) {
    b.size[i] = size[i];
    b.sstride[i] = sb[i] ? ss : 0;
    b.zstride[i] = zb[i] ? zs : 0;
    if (sb[i])
      ss *= size[i];
    if (zb[i])
      zs *= size[i];
  }
  return true;
}

__device__ __forceinline__ void offsets(const Broadcast &b, int64_t i, int64_t &so, int64_t &zo) {
  so = zo = 0;
#pragma unroll
  for (int d = kMaxDims - 1; d >= 0; --d) {
    if (d < b.nd) {
      const int64_t q = (d == 0) ? 0 : i / b.size[d];
      const int64_t c = (d == 0) ? i : i - q * b.size[d];
      so += c * b.sstride[d];
      zo += c * b.zstride[d];
      i = q;
    }
  }
}

// quantize_linear.cpp:78-95
__device__ __forceinline__ float round_mode(float v, int half_to_even) {
  const float t = round_half_away(v);
  if (half_to_even && fabsf(v - t) == 0.5f)
    return round_half_away(v * 0.5f) * 2.0f;
  return t;
}
__device__ __forceinline__ float saturate(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

struct QuantizeOp {
  int half_to_even;
  float lo, hi;
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const {
    const float t = round_mode(x / scale, half_to_even);
    return saturate(t + zp, lo, hi);
  }
};
struct DequantizeOp {
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const { return (x - zp) * scale; }
};
// dx (+)= dy / scale  and  dx (+)= dy * scale  (the zero point is not read)
struct DivGradOp {
  __device__ __forceinline__ float operator()(float dy, float scale, float) const { return dy / scale; }
};
struct MulGradOp {
  __device__ __forceinline__ float operator()(float dy, float scale, float) const { return dy * scale; }
};

// y[i] = op(x[i], scale[...], zp[...]) (+ y[i] when kAccum).  kVec: four consecutive elements per thread, all inside
// the innermost dimension (its size is a multiple of four).
template <typename Op, bool kVec, bool kAccum>
__global__ __launch_bounds__(kBlock) void broadcast_map(const float *__restrict__ x, const float *__restrict__ scale,
                                                        const float *__restrict__ zp, float *__restrict__ y,
                                                        int64_t count, Broadcast b, Op op) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < count; t += step) {
    int64_t so, zo;
    if (kVec) {
      const int64_t i = 4 * t;
      offsets(b, i, so, zo);
      const int64_t ss = b.sstride[b.nd - 1], zs = b.zstride[b.nd - 1];
      const float4_t v = *reinterpret_cast<const float4_t *>(x + i);
      float4_t o;
      o.x = op(v.x, scale[so], zp ? zp[zo] : 0.0f);
      o.y = op(v.y, scale[so + ss], zp ? zp[zo + zs] : 0.0f);
      o.z = op(v.z, scale[so + 2 * ss], zp ? zp[zo + 2 * zs] : 0.0f);
      o.w = op(v.w, scale[so + 3 * ss], zp ? zp[zo + 3 * zs] : 0.0f);
      if (kAccum) {
        const float4_t old = *reinterpret_cast<const float4_t *>(y + i);
        o.x = old.x + o.x, o.y = old.y + o.y, o.z = old.z + o.z, o.w = old.w + o.w;
      }
      __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(y + i));
    } else {
      offsets(b, t, so, zo);
      const float o = op(x[t], scale[so], zp ? zp[zo] : 0.0f);
      y[t] = kAccum ? y[t] + o : o;
    }
  }
}

// zero_point <- saturate(round(zero_point)), in place (quantize_linear.cpp:109-111)
__global__ __launch_bounds__(kBlock) void round_zero_point(float *__restrict__ zp, int64_t n, int half_to_even, float lo,
                                                           float hi) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    zp[i] = saturate(round_mode(zp[i], half_to_even), lo, hi);
}

template <typename Op>
int launch_broadcast(const float *x, const float *scale, const float *zp, float *y, const int64_t *xshape,
                     const int64_t *sshape, const int64_t *zshape, int ndim, bool accum, Op op, hipStream_t stream,
                     const char *what) {
  int64_t total = 1;
  for (int i = 0; i < ndim; ++i) {
    if (xshape[i] < 0 || (sshape[i] != 1 && sshape[i] != xshape[i]) || (zshape[i] != 1 && zshape[i] != xshape[i]))
      return fail(NBLA_HIP_ERR_VALUE, "%s: scale / zero point sizes must be 1 or match the input at dimension %d.", what,
                  i);
    total *= xshape[i];
  }
  if (total == 0)
    return NBLA_HIP_OK;
  Broadcast b;
  if (ndim > 32 || !make_broadcast(b, xshape, sshape, zshape, ndim))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "%s: more than %d alternating broadcast groups.", what, kMaxDims);
  int rc = ensure_init();
  if (rc)
    return rc;
  const bool vec = b.size[b.nd - 1] % 4 == 0 && aligned16(x) && aligned16(y);
  const int64_t count = vec ? total / 4 : total;
  int64_t blocks = ceil_div(count, (int64_t)kBlock);
  if (blocks > 1048576)
    blocks = 1048576;
#define NBLA_LAUNCH_MAP(V, A)                                                                                          \
  hipLaunchKernelGGL((broadcast_map<Op, V, A>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, scale, zp, y,      \
                     count, b, op)
  if (vec && accum)
    NBLA_LAUNCH_MAP(true, true);
  else if (vec)
    NBLA_LAUNCH_MAP(true, false);
  else if (accum)
    NBLA_LAUNCH_MAP(false, true);
  else
    NBLA_LAUNCH_MAP(false, false);
#undef NBLA_LAUNCH_MAP
  NBLA_HIP_LAUNCH_CHECK(what);
  return NBLA_HIP_OK;
}

int quantize_range(int dtype, int narrow_range, float &lo, float &hi) {
  if (dtype == NBLA_HIP_DTYPE_BYTE) {
    lo = narrow_range ? -127.0f : -128.0f, hi = 127.0f;
  } else if (dtype == NBLA_HIP_DTYPE_UBYTE) {
    lo = narrow_range ? 1.0f : 0.0f, hi = 255.0f;
  } else {
    return fail(NBLA_HIP_ERR_VALUE, "QuantizeLinear: dtype must be BYTE (%d) or UBYTE (%d), got %d.",
                NBLA_HIP_DTYPE_BYTE, NBLA_HIP_DTYPE_UBYTE, dtype);
  }
  return NBLA_HIP_OK;
}

// ------------------------------------------------------------------------------------------------------ Prune

constexpr int kBins = 2048;
struct SelectState {
  uint32_t prefix; // magnitude bits fixed so far (already shifted into place)
  uint32_t rank;   // rank of the wanted element among those sharing the prefix
  uint32_t hist[kBins];
};

// Histogram of `bits` bits at `shift` of the magnitudes whose bits above shift + bits equal the prefix.
__global__ __launch_bounds__(kBlock) void prune_histogram(const float *__restrict__ x, int64_t n,
                                                          SelectState *__restrict__ st, int shift, int bits,
                                                          int first) {
  __shared__ uint32_t h[kBins];
  for (int i = threadIdx.x; i < kBins; i += kBlock)
    h[i] = 0u;
  __syncthreads();
  const uint32_t prefix = first ? 0u : st->prefix;
  const uint32_t mask = (1u << bits) - 1u;
  const int above = shift + bits;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const uint32_t key = __float_as_uint(x[i]) & 0x7fffffffu;
    if (first || (key >> above) == (prefix >> above))
      atomicAdd(&h[(key >> shift) & mask], 1u);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kBins; i += kBlock)
    if (h[i])
      atomicAdd(&st->hist[i], h[i]);
}

// One block: find the bin holding the wanted rank, extend the prefix, clear the histogram for the next pass.
__global__ __launch_bounds__(kBlock) void prune_pick(SelectState *__restrict__ st, int shift, int bits, int first,
                                                     uint32_t rank0) {
  __shared__ uint32_t part[kBlock];
  const int per = kBins / kBlock; // 8 consecutive bins per thread
  uint32_t local[per];
  uint32_t sum = 0;
  for (int j = 0; j < per; ++j) {
    local[j] = st->hist[threadIdx.x * per + j];
    sum += local[j];
  }
  part[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t rank = first ? rank0 : st->rank;
    uint32_t before = 0;
    int t = 0;
    while (t < kBlock - 1 && before + part[t] <= rank)
      before += part[t++];
    part[0] = (uint32_t)t; // owning thread
    part[1] = before;
    part[2] = rank;
  }
  __syncthreads();
  const uint32_t owner = part[0], before = part[1], rank = part[2];
  __syncthreads();
  if (threadIdx.x == owner) {
    uint32_t acc = before;
    int j = 0;
    while (j < per - 1 && acc + local[j] <= rank)
      acc += local[j++];
    const uint32_t bin = owner * per + j;
    st->prefix = (first ? 0u : st->prefix) | (bin << shift);
    st->rank = rank - acc;
  }
  for (int j = 0; j < per; ++j)
    st->hist[threadIdx.x * per + j] = 0u;
  (void)bits;
}

__global__ __launch_bounds__(kBlock) void clear_select(SelectState *st) {
  for (int i = threadIdx.x; i < kBins; i += kBlock)
    st->hist[i] = 0u;
  if (threadIdx.x == 0)
    st->prefix = st->rank = 0u;
}

// y = (|x| < thresh) ? 0 : x with thresh = |k-th smallest| (+ 1 when rate == 1), prune.cpp:62-69
__global__ __launch_bounds__(kBlock) void prune_apply(const float *__restrict__ x, float *__restrict__ y, int64_t n4,
                                                      int64_t n, const SelectState *__restrict__ st, float add) {
  const float thresh = __uint_as_float(st->prefix) + add;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < n4; t += step) {
    const float4_t v = *reinterpret_cast<const float4_t *>(x + 4 * t);
    float4_t o;
    o.x = fabsf(v.x) < thresh ? 0.0f : v.x;
    o.y = fabsf(v.y) < thresh ? 0.0f : v.y;
    o.z = fabsf(v.z) < thresh ? 0.0f : v.z;
    o.w = fabsf(v.w) < thresh ? 0.0f : v.w;
    __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(y + 4 * t));
  }
  if (blockIdx.x == 0) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < n)
      y[i] = fabsf(x[i]) < thresh ? 0.0f : x[i];
  }
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_quantize_linear_f32(const float *x, const float *scale, float *zero_point, float *y,
                                 const int64_t *xshape, const int64_t *scale_shape, const int64_t *zero_point_shape,
                                 int ndim, int half_to_even, int narrow_range, int dtype, void *stream_) {
  float lo, hi;
  int rc = quantize_range(dtype, narrow_range, lo, hi);
  if (rc)
    return rc;
  rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  int64_t zsize = 1;
  for (int i = 0; i < ndim; ++i)
    zsize *= zero_point_shape[i];
  if (zsize > 0) {
    int64_t blocks = ceil_div(zsize, (int64_t)kBlock);
    if (blocks > 65536)
      blocks = 65536;
    hipLaunchKernelGGL(round_zero_point, dim3((unsigned)blocks), dim3(kBlock), 0, stream, zero_point, zsize,
                       half_to_even ? 1 : 0, lo, hi);
    NBLA_HIP_LAUNCH_CHECK("round_zero_point");
  }
  QuantizeOp op{half_to_even ? 1 : 0, lo, hi};
  return launch_broadcast(x, scale, zero_point, y, xshape, scale_shape, zero_point_shape, ndim, false, op, stream,
                          "QuantizeLinear");
}

int nbla_hip_dequantize_linear_f32(const float *x, const float *scale, const float *zero_point, float *y,
                                   const int64_t *xshape, const int64_t *scale_shape, const int64_t *zero_point_shape,
                                   int ndim, void *stream_) {
  return launch_broadcast(x, scale, zero_point, y, xshape, scale_shape, zero_point_shape, ndim, false, DequantizeOp(),
                          as_stream(stream_), "DequantizeLinear");
}

int nbla_hip_quantize_linear_backward_f32(const float *dy, const float *scale, float *dx, const int64_t *xshape,
                                          const int64_t *scale_shape, int ndim, int accum, void *stream_) {
  int64_t ones[32];
  if (ndim > 32)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "QuantizeLinear backward: more than 32 dimensions.");
  for (int i = 0; i < ndim; ++i)
    ones[i] = 1;
  return launch_broadcast(dy, scale, nullptr, dx, xshape, scale_shape, ones, ndim, accum != 0, DivGradOp(),
                          as_stream(stream_), "QuantizeLinear backward");
}

int nbla_hip_dequantize_linear_backward_f32(const float *dy, const float *scale, float *dx, const int64_t *xshape,
                                            const int64_t *scale_shape, int ndim, int accum, void *stream_) {
  int64_t ones[32];
  if (ndim > 32)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "DequantizeLinear backward: more than 32 dimensions.");
  for (int i = 0; i < ndim; ++i)
    ones[i] = 1;
  return launch_broadcast(dy, scale, nullptr, dx, xshape, scale_shape, ones, ndim, accum != 0, MulGradOp(),
                          as_stream(stream_), "DequantizeLinear backward");
}

size_t nbla_hip_prune_workspace_bytes(void) { return round_up(sizeof(SelectState), 256); }

int nbla_hip_prune_f32(const float *x, float *y, size_t size, float rate, void *workspace, size_t workspace_bytes,
                       void *stream_) {
  if (!(rate >= 0.0f && rate <= 1.0f))
    return fail(NBLA_HIP_ERR_VALUE, "Rate %f must be in [0, 1].", (double)rate);
  if (size == 0)
    return NBLA_HIP_OK;
  if (size > 0x7fffffffu)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "Prune: more than 2^31 - 1 elements (the reference indexes with int).");
  if (workspace_bytes < sizeof(SelectState) || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "Prune workspace too small or misaligned.");
  if (!aligned16(x) || !aligned16(y))
    return fail(NBLA_HIP_ERR_MEMORY, "Prune: x and y must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  SelectState *st = static_cast<SelectState *>(workspace);
  // prune.cpp:33-34: thresh_idx_ = (int)((x_size - 1) * rate_), an int times a float
  const int x_size = (int)size;
  const uint32_t rank = (uint32_t)(int)((x_size - 1) * rate);
  const int64_t n = (int64_t)size;
  int64_t blocks = ceil_div(n, (int64_t)kBlock * 16);
  if (blocks > 2048)
    blocks = 2048;
  if (blocks < 1)
    blocks = 1;
  hipLaunchKernelGGL(clear_select, dim3(1), dim3(kBlock), 0, stream, st);
  NBLA_HIP_LAUNCH_CHECK("clear_select");
  const int shifts[3] = {20, 10, 0}, widths[3] = {11, 10, 10};
  for (int p = 0; p < 3; ++p) {
    hipLaunchKernelGGL(prune_histogram, dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, n, st, shifts[p],
                       widths[p], p == 0 ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("prune_histogram");
    hipLaunchKernelGGL(prune_pick, dim3(1), dim3(kBlock), 0, stream, st, shifts[p], widths[p], p == 0 ? 1 : 0, rank);
    NBLA_HIP_LAUNCH_CHECK("prune_pick");
  }
  const int64_t n4 = n / 4;
  int64_t ablocks = ceil_div(n4 ? n4 : 1, (int64_t)kBlock * 4);
  hipLaunchKernelGGL(prune_apply, dim3((unsigned)ablocks), dim3(kBlock), 0, stream, x, y, n4, n, st,
                     rate == 1.0f ? 1.0f : 0.0f);
  NBLA_HIP_LAUNCH_CHECK("prune_apply");
  return NBLA_HIP_OK;
}

} // extern "C"
