// Backward passes (straight-through estimators) of FixedPointQuantize, Pow2Quantize and MinMaxQuantize:
// HBM-bound elementwise kernels (128-bit accesses) and, for the MinMaxQuantize range gradients, masked sums with a
// fixed summation order.
#include "common.hpp"
#include "quantize_common.hpp"

#include <cmath>
#include <cstring>

namespace nbla_hip {
namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;

__device__ __forceinline__ float4_t load4(const float *p) { return *reinterpret_cast<const float4_t *>(p); }
__device__ __forceinline__ void store4(float *p, float4_t v) {
  __builtin_nontemporal_store(v, reinterpret_cast<float4_t *>(p));
}

// dx[i] = op(dy[i], x[i], i) (+ dx[i] when kAccum).  `op` returns the gradient contribution; kUseX tells whether x is
// read at all.
template <typename Op, bool kAccum, bool kUseX>
__global__ __launch_bounds__(kBlock) void grad_vec4(const float *__restrict__ dy, const float *__restrict__ x,
                                                    float *__restrict__ dx, size_t n4, size_t size, Op op) {
  const size_t base = (size_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
  float4_t g[kUnroll], v[kUnroll], o[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      g[j] = load4(dy + 4 * i);
      if (kUseX)
        v[j] = load4(x + 4 * i);
      if (kAccum)
        o[j] = load4(dx + 4 * i);
    }
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      float4_t r;
      r.x = op.template apply<kAccum>(g[j].x, kUseX ? v[j].x : 0.0f, kAccum ? o[j].x : 0.0f, 4 * i);
      r.y = op.template apply<kAccum>(g[j].y, kUseX ? v[j].y : 0.0f, kAccum ? o[j].y : 0.0f, 4 * i + 1);
      r.z = op.template apply<kAccum>(g[j].z, kUseX ? v[j].z : 0.0f, kAccum ? o[j].z : 0.0f, 4 * i + 2);
      r.w = op.template apply<kAccum>(g[j].w, kUseX ? v[j].w : 0.0f, kAccum ? o[j].w : 0.0f, 4 * i + 3);
      store4(dx + 4 * i, r);
    }
  }
  if (blockIdx.x == 0) {
    const size_t i = 4 * n4 + threadIdx.x;
    if (i < size)
      dx[i] = op.template apply<kAccum>(dy[i], kUseX ? x[i] : 0.0f, kAccum ? dx[i] : 0.0f, i);
  }
}

template <typename Op, bool kAccum, bool kUseX>
__global__ __launch_bounds__(kBlock) void grad_scalar(const float *__restrict__ dy, const float *__restrict__ x,
                                                      float *__restrict__ dx, size_t size, Op op) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlock)
    dx[i] = op.template apply<kAccum>(dy[i], kUseX ? x[i] : 0.0f, kAccum ? dx[i] : 0.0f, i);
}

template <typename Op, bool kUseX>
int launch_grad(const float *dy, const float *x, float *dx, size_t size, int accum, Op op, hipStream_t stream,
                const char *what) {
  if (size == 0)
    return NBLA_HIP_OK;
  if (aligned16(dy) && aligned16(dx) && (!kUseX || aligned16(x))) {
    const size_t n4 = size / 4, tile = (size_t)kBlock * kUnroll;
    const size_t blocks = n4 ? (n4 + tile - 1) / tile : 1;
    if (accum)
      hipLaunchKernelGGL((grad_vec4<Op, true, kUseX>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, dy, x, dx, n4,
                         size, op);
    else
      hipLaunchKernelGGL((grad_vec4<Op, false, kUseX>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, dy, x, dx, n4,
                         size, op);
  } else {
    size_t blocks = (size + kBlock - 1) / kBlock;
    if (blocks > 65536)
      blocks = 65536;
    if (accum)
      hipLaunchKernelGGL((grad_scalar<Op, true, kUseX>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, dy, x, dx,
                         size, op);
    else
      hipLaunchKernelGGL((grad_scalar<Op, false, kUseX>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, dy, x, dx,
                         size, op);
  }
  NBLA_HIP_LAUNCH_CHECK(what);
  return NBLA_HIP_OK;
}

// Plain straight-through: dx (+)= dy  (fixed_point_quantize.cpp:69-78, pow2_quantize.cpp:84-93,
// min_max_quantize.cpp:285-291).
struct PassOp {
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float, float old, size_t) const {
    return kAccum ? dy + old : dy;
  }
};

// fixed_point_quantize.cpp:81-99: gradient only inside [min, max]; outside, an accumulated dx is left as it is.
struct FixedPointGradOp {
  float max_, min_;
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float x, float old, size_t) const {
    if (x > max_ || x < min_)
      return kAccum ? old : 0.0f;
    return kAccum ? old + dy : dy;
  }
};

// pow2_quantize.cpp:96-125: c = 0 where 2^round(log2|x|) > p_max (|x| at or above the calibrated cut of binade
// log2(p_max), infinity included) and, unsigned, where x < 0; dx (+)= c * dy as a product.
struct Pow2GradOp {
  uint32_t cut; // first |x| pattern whose rounded exponent exceeds log2(p_max)
  int sign;
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float x, float old, size_t) const {
    const uint32_t u = __float_as_uint(x) & 0x7fffffffu;
    float c = (u >= cut && u <= 0x7f800000u) ? 0.0f : 1.0f; // NaN: q > p_max is false
    if (!sign)
      c = (x < 0.0f) ? 0.0f : c;
    const float t = c * dy;
    return kAccum ? old + t : t;
  }
};

// min_max_quantize.cpp:262-284: mask = (x >= m') * (x <= M'), dx = mask * dy (+ dx); bounds per channel
// (element i belongs to channel (i / R1) % K).
struct MinMaxGradOp {
  const float2 *bounds; // (m', M') per channel
  int64_t K, R1;
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float x, float old, size_t i) const {
    const float2 b = bounds[K == 1 ? 0 : (int64_t)(i / R1) % K];
    const float iv0 = (x >= b.x) ? 1.0f : 0.0f, iv1 = (x <= b.y) ? 1.0f : 0.0f;
    float mask = iv0 * iv1;
    mask = mask * dy;
    return kAccum ? mask + old : mask;
  }
};

// The same mask for any pattern of kept and reduced axes: element i belongs to the kept index formed by its
// coordinates along the kept axes.
struct MinMaxGradStridedOp {
  const float2 *bounds;
  MinMaxAxes A;
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float x, float old, size_t i) const {
    int64_t k = 0;
    for (int d = 0; d < A.nkept; ++d)
      k = k * A.ksize[d] + ((int64_t)i / A.kstride[d]) % A.ksize[d];
    const float2 b = bounds[k];
    const float iv0 = (x >= b.x) ? 1.0f : 0.0f, iv1 = (x <= b.y) ? 1.0f : 0.0f;
    float mask = iv0 * iv1;
    mask = mask * dy;
    return kAccum ? mask + old : mask;
  }
};

// relu.cpp:41-49: dx (+)= (y > 0 ? dy : 0), y the forward output
struct ReluGradOp {
  template <bool kAccum> __device__ __forceinline__ float apply(float dy, float y, float old, size_t) const {
    const float t = (y > 0.0f) ? dy : 0.0f;
    return kAccum ? old + t : t;
  }
};

// ---- MinMaxQuantize range gradients
__global__ __launch_bounds__(64) void minmax_bounds(const float *__restrict__ qr_min, const float *__restrict__ ql_min,
                                                    const float *__restrict__ ql_max, const float *__restrict__ scale,
                                                    float2 *__restrict__ bounds, int64_t K) {
  const int64_t k = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (k >= K)
    return;
  float m_n, M_n;
  nudge_qr_min_max(qr_min[k], ql_min[k], ql_max[k], scale[k], m_n, M_n);
  bounds[k] = float2{m_n, M_n};
}

// Block (chunk c, channel k) adds mask * dy over tiles c, c + nchunks, ... of channel k, for both masks
// (x < m' and x > M'): per thread in index order, then lanes, wavefronts in a fixed order.
constexpr int kSumTile = kBlock * 4;
__global__ __launch_bounds__(kBlock) void minmax_range_grad_partial(const float *__restrict__ dy,
                                                                    const float *__restrict__ x,
                                                                    const float2 *__restrict__ bounds,
                                                                    float2 *__restrict__ partial, int64_t K, int64_t R1,
                                                                    int64_t tiles_per_row, int64_t tiles_per_k,
                                                                    int nchunks) {
  const int64_t k = blockIdx.y;
  const float2 b = bounds[k];
  float lo = 0.0f, hi = 0.0f;
  for (int64_t t = blockIdx.x; t < tiles_per_k; t += nchunks) {
    const int64_t r0 = t / tiles_per_row, tr = t - r0 * tiles_per_row;
    const int64_t base = (r0 * K + k) * R1;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t r1 = tr * kSumTile + j * kBlock + threadIdx.x;
      if (r1 < R1) {
        const float xv = x[base + r1], g = dy[base + r1];
        lo += ((xv < b.x) ? 1.0f : 0.0f) * g;
        hi += ((xv > b.y) ? 1.0f : 0.0f) * g;
      }
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo += __shfl_xor(lo, off);
    hi += __shfl_xor(hi, off);
  }
  __shared__ float2 s_part[kBlock / 64];
  if ((threadIdx.x & 63) == 0)
    s_part[threadIdx.x >> 6] = float2{lo, hi};
  __syncthreads();
  if (threadIdx.x == 0) {
    float2 acc = s_part[0];
    for (int w = 1; w < kBlock / 64; ++w)
      acc.x += s_part[w].x, acc.y += s_part[w].y;
    partial[k * nchunks + blockIdx.x] = acc;
  }
}

// Any pattern of kept and reduced axes: block k walks the slice of kept index k, reduced axes row-major.
__global__ __launch_bounds__(kBlock) void minmax_range_grad_strided(const float *__restrict__ dy,
                                                                    const float *__restrict__ x,
                                                                    const float2 *__restrict__ bounds,
                                                                    float2 *__restrict__ partial, MinMaxAxes A,
                                                                    int64_t R) {
  const int64_t k = blockIdx.x;
  const float2 b = bounds[k];
  int64_t base = 0, idx = k;
  for (int d = A.nkept - 1; d >= 0; --d) {
    const int64_t q = idx / A.ksize[d];
    base += (idx - q * A.ksize[d]) * A.kstride[d];
    idx = q;
  }
  float lo = 0.0f, hi = 0.0f;
  for (int64_t r = threadIdx.x; r < R; r += kBlock) {
    int64_t off = base, rem = r;
    for (int d = A.nred - 1; d >= 0; --d) {
      const int64_t q = rem / A.rsize[d];
      off += (rem - q * A.rsize[d]) * A.rstride[d];
      rem = q;
    }
    const float xv = x[off], g = dy[off];
    lo += ((xv < b.x) ? 1.0f : 0.0f) * g;
    hi += ((xv > b.y) ? 1.0f : 0.0f) * g;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo += __shfl_xor(lo, off);
    hi += __shfl_xor(hi, off);
  }
  __shared__ float2 s_part[kBlock / 64];
  if ((threadIdx.x & 63) == 0)
    s_part[threadIdx.x >> 6] = float2{lo, hi};
  __syncthreads();
  if (threadIdx.x == 0) {
    float2 acc = s_part[0];
    for (int w = 1; w < kBlock / 64; ++w)
      acc.x += s_part[w].x, acc.y += s_part[w].y;
    partial[k] = acc;
  }
}

__global__ __launch_bounds__(64) void minmax_range_grad_final(const float2 *__restrict__ partial, int nchunks,
                                                              float *__restrict__ g_min, float *__restrict__ g_max,
                                                              int accum_min, int accum_max, int64_t K) {
  const int64_t k = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (k >= K)
    return;
  float lo = 0.0f, hi = 0.0f;
  for (int c = 0; c < nchunks; ++c) {
    lo += partial[k * nchunks + c].x;
    hi += partial[k * nchunks + c].y;
  }
  if (g_min)
    g_min[k] = accum_min ? g_min[k] + lo : lo; // add2(g_qr_min, sum) :316-317
  if (g_max)
    g_max[k] = accum_max ? g_max[k] + hi : hi;
}

// ---- dx and the range sums in one pass over dy and x.
// What a launch does: dx (0: not wanted, 1: dx (+)= dy, 2: dx (+)= mask * dy), whether dx is added to, and whether
// the masked sums of dy below m' / above M' are formed.  Uniform over the grid.
struct GradMode {
  int dx_mode, accum, sums;
};

// mask * dy (+ old) as min_max_quantize.cpp:262-284 forms it
__device__ __forceinline__ float minmax_dx(float g, float xv, float old, const float2 &b, const GradMode &m) {
  float t = g;
  if (m.dx_mode == 2) {
    const float iv0 = (xv >= b.x) ? 1.0f : 0.0f, iv1 = (xv <= b.y) ? 1.0f : 0.0f;
    t = iv0 * iv1;
    t = t * g;
  }
  return m.accum ? t + old : t;
}
__device__ __forceinline__ void minmax_sums(float g, float xv, const float2 &b, float &lo, float &hi) {
  lo += ((xv < b.x) ? 1.0f : 0.0f) * g;
  hi += ((xv > b.y) ? 1.0f : 0.0f) * g;
}
// lanes, then wavefronts in a fixed order; thread 0 writes
__device__ __forceinline__ void block_sums(float lo, float hi, float2 *dst) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo += __shfl_xor(lo, off);
    hi += __shfl_xor(hi, off);
  }
  __shared__ float2 s_part[kBlock / 64];
  if ((threadIdx.x & 63) == 0)
    s_part[threadIdx.x >> 6] = float2{lo, hi};
  __syncthreads();
  if (threadIdx.x == 0) {
    float2 acc = s_part[0];
    for (int w = 1; w < kBlock / 64; ++w)
      acc.x += s_part[w].x, acc.y += s_part[w].y;
    *dst = acc;
  }
}
// The range tensors of a call; bounds(k) = (m', M') of range k as minmax_bounds forms them, for kernels whose blocks
// need one range each.
struct RangeInputs {
  const float *qr_min, *ql_min, *ql_max, *scale;
  __device__ __forceinline__ float2 bounds(int64_t k) const {
    float m_n, M_n;
    nudge_qr_min_max(qr_min[k], ql_min[k], ql_max[k], scale[k], m_n, M_n);
    return float2{m_n, M_n};
  }
};

// kN float4s per thread, all loads issued before the first store (the compiler does not move a load across a store)
template <int kN>
__device__ __forceinline__ void minmax_grad4(const float *__restrict__ dy, const float *__restrict__ x,
                                             float *__restrict__ dx, const int64_t (&at)[kN], const bool (&in)[kN],
                                             const float2 &b, const GradMode &m, float &lo, float &hi) {
  const float4_t zero = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float4_t g[kN], v[kN], o[kN];
#pragma unroll
  for (int j = 0; j < kN; ++j) {
    g[j] = in[j] ? load4(dy + at[j]) : zero;
    v[j] = (in[j] && (m.dx_mode == 2 || m.sums)) ? load4(x + at[j]) : zero;
    o[j] = (in[j] && m.dx_mode && m.accum) ? load4(dx + at[j]) : zero;
  }
#pragma unroll
  for (int j = 0; j < kN; ++j) {
    if (!in[j])
      continue;
    if (m.dx_mode) {
      float4_t r;
      r.x = minmax_dx(g[j].x, v[j].x, o[j].x, b, m), r.y = minmax_dx(g[j].y, v[j].y, o[j].y, b, m);
      r.z = minmax_dx(g[j].z, v[j].z, o[j].z, b, m), r.w = minmax_dx(g[j].w, v[j].w, o[j].w, b, m);
      store4(dx + at[j], r);
    }
    if (m.sums) {
      minmax_sums(g[j].x, v[j].x, b, lo, hi), minmax_sums(g[j].y, v[j].y, b, lo, hi);
      minmax_sums(g[j].z, v[j].z, b, lo, hi), minmax_sums(g[j].w, v[j].w, b, lo, hi);
    }
  }
}

// One range for the whole tensor (16-byte aligned): block c takes the tiles c, c + gridDim.x, ... of kBlock * 4
// float4s and leaves its sums in partial[c]; block 0 also takes the elements past the last whole float4.
__global__ __launch_bounds__(kBlock) void minmax_grad_flat(const float *__restrict__ dy, const float *__restrict__ x,
                                                           float *__restrict__ dx, int64_t n4, int64_t size,
                                                           RangeInputs q, float2 *__restrict__ partial, GradMode m) {
  const float2 b = q.bounds(0);
  float lo = 0.0f, hi = 0.0f;
  const int64_t tiles = (n4 + kBlock * 4 - 1) / (kBlock * 4);
  for (int64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
    int64_t at[4];
    bool in[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t i = t * (kBlock * 4) + j * kBlock + threadIdx.x;
      in[j] = i < n4, at[j] = 4 * i;
    }
    minmax_grad4<4>(dy, x, dx, at, in, b, m, lo, hi);
  }
  if (blockIdx.x == 0) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < size) {
      const float g = dy[i], xv = x[i];
      if (m.dx_mode)
        dx[i] = minmax_dx(g, xv, m.accum ? dx[i] : 0.0f, b, m);
      if (m.sums)
        minmax_sums(g, xv, b, lo, hi);
    }
  }
  if (m.sums)
    block_sums(lo, hi, partial + blockIdx.x);
}

// Ranges per channel, rows of R1 contiguous elements (R1 % 4 == 0, 16-byte aligned): blockIdx.x = row (r0 * K + k),
// blockIdx.y = part of the row; the sums go to partial[k * nchunks + r0 * gridDim.y + blockIdx.y], nchunks =
// R0 * gridDim.y.
__global__ __launch_bounds__(kBlock) void minmax_grad_rows(const float *__restrict__ dy, const float *__restrict__ x,
                                                           float *__restrict__ dx, int64_t K, int64_t R1,
                                                           RangeInputs q, float2 *__restrict__ partial,
                                                           int64_t nchunks, GradMode m) {
  const int64_t row = blockIdx.x, r0 = row / K, k = row - r0 * K;
  const float2 b = q.bounds(k);
  const int64_t n4 = R1 / 4, at0 = row * R1;
  float lo = 0.0f, hi = 0.0f;
  const int64_t step = (int64_t)gridDim.y * kBlock;
  for (int64_t i0 = (int64_t)blockIdx.y * kBlock + threadIdx.x; i0 < n4; i0 += 4 * step) {
    int64_t at[4];
    bool in[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      in[j] = i0 + j * step < n4, at[j] = at0 + 4 * (i0 + j * step);
    minmax_grad4<4>(dy, x, dx, at, in, b, m, lo, hi);
  }
  if (m.sums)
    block_sums(lo, hi, partial + k * nchunks + r0 * gridDim.y + blockIdx.y);
}

// The inner-kept form (MinMaxInner: lanes along the kept innermost axis), block (ko, chunk) as in the forward's
// kernels of this form; the sums of column w go to partial[(ko * Wk + w) * nchunks + chunk].
template <int kVec>
__global__ __launch_bounds__(kBlock) void minmax_grad_inner(const float *__restrict__ dy, const float *__restrict__ x,
                                                            float *__restrict__ dx, MinMaxAxes A, MinMaxInner I,
                                                            int nchunks, const float2 *__restrict__ bounds,
                                                            float2 *__restrict__ partial, GradMode m) {
  __shared__ float2 s_part[kBlock / 64][64][kVec];
  const int64_t ko = blockIdx.x;
  const int chunk = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tw = I.tw, rows_per_step = kBlock / tw;
  const int cw = tid & (tw - 1), slot = tid / tw;
  const InnerWalk W = inner_walk(x, A, I, ko, chunk, nchunks);
  constexpr int kRows = 4; // rows in flight per lane
  for (int64_t w0 = 0; w0 < I.Wk; w0 += (int64_t)tw * kVec) {
    const int64_t wcol = w0 + (int64_t)cw * kVec;
    const bool col_in = wcol < I.Wk;
    float2 b[kVec];
    float lo[kVec], hi[kVec];
#pragma unroll
    for (int c = 0; c < kVec; ++c) {
      b[c] = bounds[ko * I.Wk + (col_in ? wcol + c : 0)];
      lo[c] = hi[c] = 0.0f;
    }
    for (int64_t ro = W.ro_begin; ro < W.ro_end; ++ro) {
      const int64_t off = (W.base - x) + (A.nred > 1 ? strided_offset(ro, A.nred - 1, A.rsize, A.rstride) : 0) + wcol;
      for (int64_t ri0 = 0; ri0 < I.Rin; ri0 += kRows * rows_per_step) {
        InnerRow<kVec> g[kRows], v[kRows], o[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          const bool in = col_in && ri < I.Rin;
          const int64_t at = off + ri * I.rin_stride;
          if (in)
            g[j].load(dy + at);
          else
            g[j].fill(0.0f);
          if (in && (m.dx_mode == 2 || m.sums))
            v[j].load(x + at);
          else
            v[j].fill(0.0f);
          if (in && m.dx_mode && m.accum)
            o[j].load(dx + at);
          else
            o[j].fill(0.0f);
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          if (!(col_in && ri < I.Rin))
            continue;
          if (m.dx_mode) {
            float *dst = dx + off + ri * I.rin_stride;
            float r[kVec];
#pragma unroll
            for (int c = 0; c < kVec; ++c)
              r[c] = minmax_dx(g[j].v[c], v[j].v[c], o[j].v[c], b[c], m);
            if (kVec == 4)
              store4(dst, float4_t{r[0], r[1 % kVec], r[2 % kVec], r[3 % kVec]});
            else
              __builtin_nontemporal_store(r[0], dst);
          }
          if (m.sums) {
#pragma unroll
            for (int c = 0; c < kVec; ++c)
              minmax_sums(g[j].v[c], v[j].v[c], b[c], lo[c], hi[c]);
          }
        }
      }
    }
    if (!m.sums) // uniform
      continue;
    // fold the row slots that share a column: across the lanes of a wavefront, then across the wavefronts
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      for (int off = 32; off >= tw; off >>= 1) {
        lo[c] += __shfl_xor(lo[c], off);
        hi[c] += __shfl_xor(hi[c], off);
      }
    __syncthreads(); // the previous pass's partial results have been read
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      s_part[wave][lane][c] = float2{lo[c], hi[c]};
    __syncthreads();
    if (tid < tw && col_in) {
#pragma unroll
      for (int c = 0; c < kVec; ++c) {
        float2 acc = s_part[0][tid][c];
        for (int w = 1; w < kBlock / 64; ++w)
          acc.x += s_part[w][tid][c].x, acc.y += s_part[w][tid][c].y;
        partial[(ko * I.Wk + wcol + c) * nchunks + chunk] = acc;
      }
    }
  }
}

// The row form (MinMaxRows: the innermost axis reduced, T lanes per run of Rin elements), block (tile of 256 / T kept
// indices, chunk) as in the forward's kernels of this form; the sums of kept index k go to partial[k * nchunks + chunk].
template <int kVec>
__global__ __launch_bounds__(kBlock) void minmax_grad_rowform(const float *__restrict__ dy, const float *__restrict__ x,
                                                              float *__restrict__ dx, MinMaxAxes A, MinMaxRows R, int T,
                                                              int nchunks, const float2 *__restrict__ bounds,
                                                              float2 *__restrict__ partial, GradMode m) {
  const int tid = threadIdx.x, li = tid & (T - 1), slot = tid / T, rps = kBlock / T;
  const int64_t k = (int64_t)blockIdx.x * rps + slot;
  const bool k_in = k < R.K;
  const int chunk = blockIdx.y;
  const RowWalk W = row_walk(R, chunk, nchunks);
  const int64_t base = strided_offset(k_in ? k : 0, A.nkept, A.ksize, A.kstride);
  const float2 b = bounds[k_in ? k : 0];
  float lo = 0.0f, hi = 0.0f;
  constexpr int kRows = 4; // outer reduced indices in flight per lane
  for (int64_t ro = W.ro_begin; ro < W.ro_end; ro += kRows) {
    int64_t off[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j)
      off[j] = base + ((A.nred > 1 && ro + j < W.ro_end) ? strided_offset(ro + j, A.nred - 1, A.rsize, A.rstride) : 0);
    for (int64_t ri0 = 0; ri0 < R.Rin; ri0 += (int64_t)T * kVec) {
      const int64_t ri = ri0 + (int64_t)li * kVec;
      InnerRow<kVec> g[kRows], v[kRows], o[kRows];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        const bool in = k_in && ro + j < W.ro_end && ri < R.Rin;
        const int64_t at = off[j] + ri;
        if (in)
          g[j].load(dy + at);
        else
          g[j].fill(0.0f);
        if (in && (m.dx_mode == 2 || m.sums))
          v[j].load(x + at);
        else
          v[j].fill(0.0f);
        if (in && m.dx_mode && m.accum)
          o[j].load(dx + at);
        else
          o[j].fill(0.0f);
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (!(k_in && ro + j < W.ro_end && ri < R.Rin))
          continue;
        if (m.dx_mode) {
          float *dst = dx + off[j] + ri;
          float r[kVec];
#pragma unroll
          for (int c = 0; c < kVec; ++c)
            r[c] = minmax_dx(g[j].v[c], v[j].v[c], o[j].v[c], b, m);
          if (kVec == 4)
            store4(dst, float4_t{r[0], r[1 % kVec], r[2 % kVec], r[3 % kVec]});
          else
            __builtin_nontemporal_store(r[0], dst);
        }
        if (m.sums) {
#pragma unroll
          for (int c = 0; c < kVec; ++c)
            minmax_sums(g[j].v[c], v[j].v[c], b, lo, hi);
        }
      }
    }
  }
  if (!m.sums)
    return;
  for (int o = T >> 1; o >= 1; o >>= 1) {
    lo += __shfl_xor(lo, o);
    hi += __shfl_xor(hi, o);
  }
  if (li == 0 && k_in)
    partial[k * nchunks + chunk] = float2{lo, hi};
}

// A wavefront per range: lane l adds the partial sums l, l + 64, ... in order, then the lanes are added up.
__global__ __launch_bounds__(64) void minmax_range_grad_final_wave(const float2 *__restrict__ partial, int64_t nchunks,
                                                                   float *__restrict__ g_min, float *__restrict__ g_max,
                                                                   int accum_min, int accum_max) {
  const int64_t k = blockIdx.x;
  float lo = 0.0f, hi = 0.0f;
  for (int64_t c = threadIdx.x; c < nchunks; c += 64) {
    const float2 p = partial[k * nchunks + c];
    lo += p.x, hi += p.y;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo += __shfl_xor(lo, off);
    hi += __shfl_xor(hi, off);
  }
  if (threadIdx.x == 0) {
    if (g_min)
      g_min[k] = accum_min ? g_min[k] + lo : lo;
    if (g_max)
      g_max[k] = accum_max ? g_max[k] + hi : hi;
  }
}

// Which one-pass kernel a shape can take (the pointers' alignment decides at the call) and the partial sums each
// leaves per range; the workspace holds the largest.
struct RangeGradPlan {
  MinMaxLayout L;
  int64_t tiles_per_row, tiles_per_k;
  int nchunks;          // of the two-pass kernels
  bool inner;           // the lanes-along-the-kept-axis form applies
  MinMaxAxes axes;
  MinMaxInner I;
  int inner_chunks;
  bool rows;            // the runs-along-the-innermost-reduced-axis form applies
  MinMaxRows R;
  int row_form_chunks;
  int64_t flat_chunks;  // K == 1
  int64_t row_parts;    // rows form (R1 % 4 == 0, R1 >= 256): blocks along a row; partial sums per range = R0 * row_parts
  size_t bounds_bytes, partial_bytes;
};

RangeGradPlan make_range_plan(const int64_t *xshape, int ndim, const int64_t *qshape) {
  RangeGradPlan P;
  P.L = collapse(xshape, ndim, qshape);
  P.tiles_per_row = (P.L.R1 + kSumTile - 1) / kSumTile;
  P.tiles_per_k = P.tiles_per_row * P.L.R0;
  int64_t chunks = 1024 / (P.L.K < 1024 ? P.L.K : 1024);
  if (chunks < 1)
    chunks = 1;
  if (chunks > P.tiles_per_k)
    chunks = P.tiles_per_k;
  if (chunks < 1)
    chunks = 1;
  if (!P.L.ok)
    chunks = 1; // the strided kernel folds a whole slice per block
  P.nchunks = (int)chunks;
  int64_t most = chunks;
  P.inner = false;
  P.inner_chunks = 1;
  if ((!P.L.ok || trailing_kept(P.L)) && split_axes(xshape, ndim, qshape, P.axes)) {
    P.I = inner_form(P.axes);
    if (P.I.ok) {
      P.inner = true;
      P.inner_chunks = (int)inner_chunks(P.I);
      most = most > P.inner_chunks ? most : P.inner_chunks;
    }
  }
  P.rows = false;
  P.row_form_chunks = 1;
  if (!P.inner && (!P.L.ok || short_rows(P.L)) && split_axes(xshape, ndim, qshape, P.axes)) {
    P.R = row_form(P.axes);
    if (P.R.ok) {
      P.rows = true;
      P.row_form_chunks = (int)row_chunks(P.R);
      most = most > P.row_form_chunks ? most : P.row_form_chunks;
    }
  }
  P.flat_chunks = 0;
  if (P.L.ok && P.L.K == 1) {
    const int64_t tiles = (P.L.total / 4 + kBlock * 4 - 1) / (kBlock * 4);
    P.flat_chunks = tiles < 1 ? 1 : (tiles > 1024 ? 1024 : tiles);
    most = most > P.flat_chunks ? most : P.flat_chunks;
  }
  P.row_parts = 0;
  if (P.L.ok && P.L.K > 1 && P.L.R1 % 4 == 0 && P.L.R1 >= 256 && P.L.R0 * P.L.K <= 0x7fffffffll) {
    // about 4096 blocks; a block takes at least one float4 per thread
    int64_t parts = (4096 + P.L.R0 * P.L.K - 1) / (P.L.R0 * P.L.K);
    const int64_t longest = (P.L.R1 / 4 + kBlock - 1) / kBlock;
    if (parts > longest)
      parts = longest;
    if (parts > 64)
      parts = 64;
    P.row_parts = parts < 1 ? 1 : parts;
    most = most > P.L.R0 * P.row_parts ? most : P.L.R0 * P.row_parts;
  }
  P.bounds_bytes = round_up((size_t)P.L.K * sizeof(float2), 256);
  P.partial_bytes = round_up((size_t)P.L.K * most * sizeof(float2), 256);
  return P;
}

// g_qr_min / g_qr_max from `chunks` partial sums per range
void launch_range_final(const float2 *partial, int64_t chunks, float *g_min, float *g_max, int accum_min,
                        int accum_max, int64_t K, hipStream_t stream) {
  if (chunks <= 16 && K >= 64)
    hipLaunchKernelGGL(minmax_range_grad_final, dim3((unsigned)((K + 63) / 64)), dim3(64), 0, stream, partial,
                       (int)chunks, g_min, g_max, accum_min, accum_max, K);
  else
    hipLaunchKernelGGL(minmax_range_grad_final_wave, dim3((unsigned)K), dim3(64), 0, stream, partial, chunks, g_min,
                       g_max, accum_min, accum_max);
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_fixed_point_quantize_backward_f32(const float *dy, const float *x, float *dx, size_t size, int sign, int n,
                                               float delta, int ste_fine_grained, int accum, void *stream) {
  if (!(n > 0 && delta > 0.))
    return fail(NBLA_HIP_ERR_VALUE, "Both bit width and delta should be positive.");
  const int nn = sign ? n - 1 : n;
  if (!(nn > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive when considering sign (1bit).");
  int rc = ensure_init();
  if (rc)
    return rc;
  if (!ste_fine_grained)
    return launch_grad<PassOp, false>(dy, x, dx, size, accum, PassOp(), as_stream(stream), "quantize backward");
  const float max_ = (float)((std::pow(2, nn) - 1) * delta);
  const float min_ = sign ? (float)(-max_) : 0.0f;
  return launch_grad<FixedPointGradOp, true>(dy, x, dx, size, accum, FixedPointGradOp{max_, min_}, as_stream(stream),
                                             "fixed_point_quantize backward");
}

int nbla_hip_pow2_quantize_backward_f32(const float *dy, const float *x, float *dx, size_t size, int sign,
                                        int with_zero, int n, int m, int ste_fine_grained, int accum, void *stream) {
  if (!(n > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive.");
  int nn = sign ? n - 1 : n;
  nn = with_zero ? nn - 1 : nn;
  if (!(nn > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive when considering zero (1bit) and sign (1bit).");
  if (m > 127 || m < -149)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "2^%d is outside the finite non-zero fp32 range.", m);
  int rc = ensure_init();
  if (rc)
    return rc;
  if (!ste_fine_grained)
    return launch_grad<PassOp, false>(dy, x, dx, size, accum, PassOp(), as_stream(stream), "quantize backward");
  uint32_t table[kNumBinades];
  rc = nbla_hip_cut_table(kCutPow2Round, table);
  if (rc)
    return rc;
  Pow2GradOp op;
  op.cut = table[m + 149]; // round(log2 a) steps from m to m + 1 at the cut of binade m
  op.sign = sign;
  return launch_grad<Pow2GradOp, true>(dy, x, dx, size, accum, op, as_stream(stream), "pow2_quantize backward");
}

int nbla_hip_relu_backward_f32(const float *dy, const float *y, float *dx, size_t size, int accum, void *stream) {
  int rc = ensure_init();
  if (rc)
    return rc;
  return launch_grad<ReluGradOp, true>(dy, y, dx, size, accum, ReluGradOp(), as_stream(stream), "relu backward");
}

size_t nbla_hip_min_max_quantize_backward_workspace_bytes(const int64_t *xshape, int ndim, const int64_t *qshape) {
  const RangeGradPlan P = make_range_plan(xshape, ndim, qshape);
  return P.bounds_bytes + P.partial_bytes;
}

int nbla_hip_min_max_quantize_backward_f32(const float *dy, const float *x, float *dx, const int64_t *xshape, int ndim,
                                           const int64_t *qshape, const float *qr_min, const float *qr_max,
                                           const float *ql_min, const float *ql_max, const float *scale,
                                           float *g_qr_min, float *g_qr_max, int ste_fine_grained, int x_min_max,
                                           int ema, int accum_x, int accum_min, int accum_max, void *workspace,
                                           size_t workspace_bytes, void *stream_) {
  (void)qr_max;
  for (int i = 0; i < ndim; ++i)
    if (qshape[i] != 1 && qshape[i] != xshape[i])
      return fail(NBLA_HIP_ERR_VALUE, "q tensors must have size 1 or the size of x along every axis (axis %d).", i);
  const RangeGradPlan P = make_range_plan(xshape, ndim, qshape);
  MinMaxAxes axes;
  if (!P.L.ok && !split_axes(xshape, ndim, qshape, axes))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "more than eight kept or eight reduced axes of size above one.");
  if (P.L.K > 0x7fffffffll && (!P.L.ok || P.inner || P.rows))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "more than 2^31 - 1 quantization ranges.");
  if (P.L.total == 0)
    return NBLA_HIP_OK;
  if (workspace_bytes < P.bounds_bytes + P.partial_bytes || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "min_max_quantize backward workspace too small or misaligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  const bool range_grads = !(x_min_max || ema) && (g_qr_min || g_qr_max);
  float2 *bounds = static_cast<float2 *>(workspace);
  float2 *partial = reinterpret_cast<float2 *>(static_cast<char *>(workspace) + P.bounds_bytes);
  // dx and the range sums in one pass over dy and x, where a kernel of that kind covers the layout (a plain copy of dy
  // and the per-tensor mask without sums are as fast on the element-wise kernels below)
  const GradMode mode{dx ? (ste_fine_grained ? 2 : 1) : 0, accum_x, range_grads ? 1 : 0};
  const bool wanted = range_grads || (mode.dx_mode == 2 && P.L.K > 1);
  const bool vec = aligned16(dy) && aligned16(x) && (!dx || aligned16(dx));
  const bool one_range_per_block = wanted && !P.inner && !P.rows && vec && (P.flat_chunks || P.row_parts);
  if (((dx && ste_fine_grained) || range_grads) && !one_range_per_block) {
    hipLaunchKernelGGL(minmax_bounds, dim3((unsigned)((P.L.K + 63) / 64)), dim3(64), 0, stream, qr_min, ql_min, ql_max,
                       scale, bounds, P.L.K);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward bounds");
  }
  const RangeInputs ranges{qr_min, ql_min, ql_max, scale};
  if (wanted && P.inner) {
    MinMaxInner I = P.I;
    const bool quads = I.Wk % 4 == 0 && vec;
    if (quads) {
      I.tw = 1;
      while (I.tw < 64 && I.tw * 4 < I.Wk)
        I.tw *= 2;
    }
    const dim3 grid((unsigned)I.Ko, (unsigned)P.inner_chunks);
    if (quads)
      hipLaunchKernelGGL(minmax_grad_inner<4>, grid, dim3(kBlock), 0, stream, dy, x, dx, P.axes, I, P.inner_chunks,
                         bounds, partial, mode);
    else
      hipLaunchKernelGGL(minmax_grad_inner<1>, grid, dim3(kBlock), 0, stream, dy, x, dx, P.axes, I, P.inner_chunks,
                         bounds, partial, mode);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward");
    if (range_grads) {
      launch_range_final(partial, P.inner_chunks, g_qr_min, g_qr_max, accum_min, accum_max, P.L.K, stream);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
    }
    return NBLA_HIP_OK;
  }
  if (wanted && P.rows) {
    const bool quads = P.R.Rin % 4 == 0 && vec;
    const int T = row_lanes(P.R, quads ? 4 : 1);
    const int64_t rps = kBlock / T;
    const dim3 grid((unsigned)((P.R.K + rps - 1) / rps), (unsigned)P.row_form_chunks);
    if (quads)
      hipLaunchKernelGGL(minmax_grad_rowform<4>, grid, dim3(kBlock), 0, stream, dy, x, dx, P.axes, P.R, T,
                         P.row_form_chunks, bounds, partial, mode);
    else
      hipLaunchKernelGGL(minmax_grad_rowform<1>, grid, dim3(kBlock), 0, stream, dy, x, dx, P.axes, P.R, T,
                         P.row_form_chunks, bounds, partial, mode);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward");
    if (range_grads) {
      launch_range_final(partial, P.row_form_chunks, g_qr_min, g_qr_max, accum_min, accum_max, P.L.K, stream);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
    }
    return NBLA_HIP_OK;
  }
  if (wanted && P.flat_chunks && vec) {
    hipLaunchKernelGGL(minmax_grad_flat, dim3((unsigned)P.flat_chunks), dim3(kBlock), 0, stream, dy, x, dx,
                       P.L.total / 4, P.L.total, ranges, partial, mode);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward");
    launch_range_final(partial, P.flat_chunks, g_qr_min, g_qr_max, accum_min, accum_max, 1, stream);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
    return NBLA_HIP_OK;
  }
  if (wanted && P.row_parts && vec) {
    const int64_t chunks = P.L.R0 * P.row_parts;
    hipLaunchKernelGGL(minmax_grad_rows, dim3((unsigned)(P.L.R0 * P.L.K), (unsigned)P.row_parts), dim3(kBlock), 0,
                       stream, dy, x, dx, P.L.K, P.L.R1, ranges, partial, chunks, mode);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward");
    if (range_grads) {
      launch_range_final(partial, chunks, g_qr_min, g_qr_max, accum_min, accum_max, P.L.K, stream);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
    }
    return NBLA_HIP_OK;
  }
  if (dx) {
    if (ste_fine_grained && !P.L.ok) {
      MinMaxGradStridedOp op{bounds, axes};
      rc = launch_grad<MinMaxGradStridedOp, true>(dy, x, dx, (size_t)P.L.total, accum_x, op, stream,
                                                  "min_max_quantize backward");
    } else if (ste_fine_grained) {
      MinMaxGradOp op{bounds, P.L.K, P.L.R1};
      rc = launch_grad<MinMaxGradOp, true>(dy, x, dx, (size_t)P.L.total, accum_x, op, stream, "min_max_quantize backward");
    } else {
      rc = launch_grad<PassOp, false>(dy, x, dx, (size_t)P.L.total, accum_x, PassOp(), stream, "quantize backward");
    }
    if (rc)
      return rc;
  }
  if (range_grads && !P.L.ok) {
    hipLaunchKernelGGL(minmax_range_grad_strided, dim3((unsigned)P.L.K), dim3(kBlock), 0, stream, dy, x, bounds, partial,
                       axes, P.L.R1);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range sums");
    hipLaunchKernelGGL(minmax_range_grad_final, dim3((unsigned)((P.L.K + 63) / 64)), dim3(64), 0, stream, partial, 1,
                       g_qr_min, g_qr_max, accum_min, accum_max, P.L.K);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
  } else if (range_grads) {
    hipLaunchKernelGGL(minmax_range_grad_partial, dim3((unsigned)P.nchunks, (unsigned)P.L.K), dim3(kBlock), 0, stream,
                       dy, x, bounds, partial, P.L.K, P.L.R1, P.tiles_per_row, P.tiles_per_k, P.nchunks);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range sums");
    hipLaunchKernelGGL(minmax_range_grad_final, dim3((unsigned)((P.L.K + 63) / 64)), dim3(64), 0, stream, partial,
                       P.nchunks, g_qr_min, g_qr_max, accum_min, accum_max, P.L.K);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize backward range gradients");
  }
  return NBLA_HIP_OK;
}

} // extern "C"
