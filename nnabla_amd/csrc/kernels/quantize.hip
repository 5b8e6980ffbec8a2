// Elementwise quantizers (FixedPointQuantize, Pow2Quantize, MinMaxQuantize) as
// HBM-bound gfx950 kernels: 128-bit coalesced loads/stores, every fp32
// operation rounded on its own (the file is compiled with -ffp-contract=off and
// correctly rounded division), wavefront-shuffle reductions for the min/max.
#include "common.hpp"
#include "quantize_common.hpp"

#include <atomic>

#include <cmath>
#include <cstring>
#include <mutex>

namespace nbla_hip {
namespace {

constexpr int kBlock = 256;  // threads per block: 4 wavefronts
constexpr int kUnroll = 4;   // float4 per thread per block tile (large inputs)
constexpr int kTile = kBlock * kUnroll; // float4 per block at full unroll


// Streaming access pattern that measured best on MI355X for a read-once/write-once map: ordinary 128-bit loads,
// nontemporal 128-bit stores.
__device__ __forceinline__ float4_t load4(const float *p) { return *reinterpret_cast<const float4_t *>(p); }
__device__ __forceinline__ void store4(float *p, float4_t v) {
  __builtin_nontemporal_store(v, reinterpret_cast<float4_t *>(p));
}

// Generic driver: applies `op` (a functor float -> float) to `size` elements.
// The vector body covers size/4 float4s; the tail (size % 4) is done by block 0.
template <typename Op, int kUnroll> __global__ __launch_bounds__(kBlock) void map_vec4(const float *__restrict__ x, float *__restrict__ y, size_t n4, size_t size, Op op) {
  op.prepare();
  const size_t base = (size_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
  float4_t v[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4)
      v[j] = load4(x + 4 * i);
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      float4_t r;
      if constexpr (Op::kFour) {
        r = op.four(v[j]);
      } else {
        r.x = op(v[j].x);
        r.y = op(v[j].y);
        r.z = op(v[j].z);
        r.w = op(v[j].w);
      }
      store4(y + 4 * i, r);
    }
  }
  if (blockIdx.x == 0) {
    const size_t i = 4 * n4 + threadIdx.x;
    if (i < size)
      y[i] = op(x[i]);
  }
}

// Fallback for pointers that are not 16-byte aligned.
template <typename Op> __global__ __launch_bounds__(kBlock) void map_scalar(const float *__restrict__ x, float *__restrict__ y, size_t size, Op op) {
  op.prepare();
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < size; i += (size_t)gridDim.x * kBlock)
    y[i] = op(x[i]);
}

template <typename Op> int launch_map(const float *x, float *y, size_t size, Op op, hipStream_t stream, const char *what) {
  if (size == 0)
    return NBLA_HIP_OK;
  if (aligned16(x) && aligned16(y)) {
    const size_t n4 = size / 4;
    // inputs too small to give every CU several 4-deep blocks get one float4 per thread instead
    if (n4 < (size_t)kBlock * kUnroll * 2048) {
      const size_t blocks = n4 ? (n4 + kBlock - 1) / kBlock : 1;
      hipLaunchKernelGGL((map_vec4<Op, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, n4, size, op);
    } else {
      const size_t tile = (size_t)kBlock * kUnroll;
      const size_t blocks = (n4 + tile - 1) / tile;
      hipLaunchKernelGGL((map_vec4<Op, kUnroll>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, n4, size, op);
    }
  } else {
    size_t blocks = (size + kBlock - 1) / kBlock;
    if (blocks > 65536)
      blocks = 65536;
    hipLaunchKernelGGL(map_scalar<Op>, dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, size, op);
  }
  NBLA_HIP_LAUNCH_CHECK(what);
  return NBLA_HIP_OK;
}

// ------------------------------------------------------------------ FixedPoint
// fixed_point_quantize.cpp:53-65.  q = |x| / delta is an fp32 divide; adding 0.5
// in double and truncating equals trunc(q) + (q - trunc(q) >= 0.5), all exact in
// fp32; the product with delta is one fp32 multiply.  When delta is a power of
// two the divide is replaced by the (bit-identical) multiply with 1/delta.
template <bool kPow2Delta> struct FixedPointOp {
  static constexpr bool kFour = false;
  float max_, min_, delta, inv_delta;
  __device__ __forceinline__ void prepare() {}
  __device__ __forceinline__ float operator()(float x) const {
    if (x > max_)
      return max_;
    if (x < min_)
      return min_;
    const float a = fabsf(x);
    const float q = kPow2Delta ? a * inv_delta : a / delta;
    const float t = truncf(q);
    const float k = (q - t >= 0.5f) ? t + 1.0f : t;
    const float y = k * delta;
    return (x < 0.0f) ? -y : y;
  }
};

// ------------------------------------------------------------------------ Pow2
// pow2_quantize.cpp:55-81.  r = roundf(log2f(|x|)) comes from the calibrated
// per-binade cut (staged in LDS); 2^r, the clamps and the sign are exact.
struct Pow2Op {
  static constexpr bool kFour = false;
  const uint32_t *cuts; // device table, kNumBinades entries
  float p_max, p_min, thr;
  int e_max, e_min; // log2 of p_max / p_min
  int sign, with_zero;
  __device__ __forceinline__ void prepare() {
    __shared__ uint32_t s_cut[kNumBinades];
    for (int i = threadIdx.x; i < kNumBinades; i += blockDim.x)
      s_cut[i] = cuts[i];
    __syncthreads();
    lds = s_cut;
  }
  const uint32_t *lds;
  __device__ __forceinline__ float operator()(float x) const {
    const uint32_t u = __float_as_uint(x) & 0x7fffffffu;
    const float a = __uint_as_float(u);
    float q;
    if (u > 0x7f800000u) {
      q = a; // NaN propagates through every comparison of the reference
    } else {
      int r;
      if (u == 0u)
        r = -100000; // log2f(0) = -inf -> 2^-inf = 0, below every p_min
      else if (u == 0x7f800000u)
        r = 100000;
      else {
        const int idx = binade_of(u);
        r = binade_exponent(idx) + (u >= lds[idx] ? 1 : 0);
      }
      if (r > e_max)
        q = p_max;
      else if (r < e_min)
        q = with_zero ? ((a < thr) ? 0.0f : p_min) : p_min;
      else
        q = pow2_int(r);
    }
    const bool neg = x < 0.0f;
    if (sign)
      return neg ? -q : q;
    return neg ? (with_zero ? 0.0f : p_min) : q;
  }
};

// Pow2Quantize with few levels (2^n' <= 8): |x| as a bit pattern is compared against the level boundaries
// directly.  roundf(log2f(a)) is a non-decreasing step function of a, so level e starts at the calibrated cut of
// binade e-1; with_zero adds the boundary p_min * 2^-0.5 below which the result is 0.  The result is the value of
// the last boundary at or below |x| (positive floats order like their bit patterns).
template <int kLevels> struct Pow2SmallOp {
  static constexpr bool kFour = true;
  uint32_t bound[kLevels]; // ascending; unused entries 0xffffffff
  float value[kLevels];    // result from bound[j] on
  float base;              // result below bound[0]
  float neg_value;         // result for x < 0 when unsigned
  int sign;
  __device__ __forceinline__ void prepare() {}
  __device__ __forceinline__ float operator()(float x) const {
    const uint32_t u = __float_as_uint(x) & 0x7fffffffu;
    float q = base;
#pragma unroll
    for (int j = 0; j < kLevels; ++j)
      q = (u >= bound[j]) ? value[j] : q;
    q = (u > 0x7f800000u) ? __uint_as_float(u) : q; // NaN propagates through every comparison of the reference
    const bool neg = x < 0.0f;
    if (sign)
      return neg ? -q : q;
    return neg ? neg_value : q;
  }
  // Four values at once: the NaN test is made on the largest of the four magnitudes (one rare branch instead of a
  // compare and a select per value); the rest is the chain above.
  __device__ __forceinline__ float4_t four(float4_t x) const {
    uint32_t u[4];
    float4_t r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      u[e] = __float_as_uint(x[e]) & 0x7fffffffu;
      float q = base;
#pragma unroll
      for (int j = 0; j < kLevels; ++j)
        q = (u[e] >= bound[j]) ? value[j] : q;
      const bool neg = x[e] < 0.0f;
      r[e] = sign ? (neg ? -q : q) : (neg ? neg_value : q);
    }
    const uint32_t top = max(max(u[0], u[1]), max(u[2], u[3]));
    if (top > 0x7f800000u) { // a NaN among the four: it propagates through every comparison of the reference
#pragma unroll
      for (int e = 0; e < 4; ++e)
        r[e] = (u[e] > 0x7f800000u) ? __uint_as_float(u[e]) : r[e];
    }
    return r;
  }
};

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_fixed_point_quantize_f32(const float *x, float *y, size_t size, int sign, int n, float delta,
                                      void *stream) {
  if (!(n > 0 && delta > 0.))
    return fail(NBLA_HIP_ERR_VALUE, "Both bit width and delta should be positive.");
  const int nn = sign ? n - 1 : n;
  if (!(nn > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive when considering sign (1bit).");
  if (nn > 30)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "bit widths above 30 overflow the reference's int conversion.");
  int rc = ensure_init();
  if (rc)
    return rc;
  // fixed_point_quantize.cpp:38-40: double arithmetic, stored to float members
  const float max_ = (float)((std::pow(2, nn) - 1) * delta);
  const float min_ = sign ? (float)(-max_) : 0.0f;
  int exp2 = 0;
  const bool pow2_delta = std::frexp(delta, &exp2) == 0.5f && std::isnormal(1.0f / delta) && std::isnormal(delta);
  if (pow2_delta) {
    FixedPointOp<true> op{max_, min_, delta, 1.0f / delta};
    return launch_map(x, y, size, op, as_stream(stream), "fixed_point_quantize");
  }
  FixedPointOp<false> op{max_, min_, delta, 0.0f};
  return launch_map(x, y, size, op, as_stream(stream), "fixed_point_quantize");
}

int nbla_hip_pow2_quantize_f32(const float *x, float *y, size_t size, int sign, int with_zero, int n, int m,
                               void *stream) {
  if (!(n > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive.");
  int nn = sign ? n - 1 : n;
  nn = with_zero ? nn - 1 : nn;
  if (!(nn > 0))
    return fail(NBLA_HIP_ERR_VALUE, "bit width should be positive when considering zero (1bit) and sign (1bit).");
  if (nn > 9)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "more than 2^9 power-of-two levels leave the fp32 exponent range.");
  const int e_max = m, e_min = m - ((1 << nn) - 1);
  if (e_max > 127 || e_min < -149)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "2^%d .. 2^%d is outside the finite non-zero fp32 range.", e_min, e_max);
  int rc = ensure_init();
  if (rc)
    return rc;
  if (nn <= 3) { // up to eight levels: boundaries and level values travel as kernel arguments
    uint32_t table[kNumBinades];
    rc = nbla_hip_cut_table(kCutPow2Round, table);
    if (rc)
      return rc;
    const int levels = 1 << nn;
    const float p_min = (float)std::pow(2., e_min);
    const float thr = (float)((float)p_min * std::pow(2., -0.5)); // pow2_quantize.cpp:39 (float member times double)
    uint32_t bound[8];
    float value[8];
    int count = 0;
    if (with_zero) { // p_min where r >= e_min (from the cut of binade e_min-1 on) or |x| >= thr; 0 below both
      uint32_t thr_bits;
      std::memcpy(&thr_bits, &thr, sizeof(thr_bits));
      const int binade = (e_min - 1) + 149;
      const uint32_t cut = binade >= 0 ? table[binade] : 1u;
      bound[count] = thr_bits < cut ? thr_bits : cut;
      value[count++] = p_min;
    }
    for (int j = 1; j < levels; ++j) {
      const int binade = (e_min + j - 1) + 149; // the cut where r steps from e_min+j-1 to e_min+j
      // below the smallest subnormal binade every positive value already rounds to >= -149
      bound[count] = binade >= 0 ? table[binade] : 1u;
      value[count++] = (float)std::pow(2., e_min + j);
    }
    auto fill = [&](auto &op) {
      constexpr int cap = (int)(sizeof(op.bound) / sizeof(op.bound[0]));
      for (int j = 0; j < cap; ++j) {
        op.bound[j] = j < count ? bound[j] : 0xffffffffu;
        op.value[j] = j < count ? value[j] : 0.0f;
      }
      op.base = with_zero ? 0.0f : p_min;
      op.neg_value = with_zero ? 0.0f : p_min;
      op.sign = sign;
    };
    if (count <= 2) {
      Pow2SmallOp<2> op;
      fill(op);
      return launch_map(x, y, size, op, as_stream(stream), "pow2_quantize");
    }
    if (count <= 4) {
      Pow2SmallOp<4> op;
      fill(op);
      return launch_map(x, y, size, op, as_stream(stream), "pow2_quantize");
    }
    Pow2SmallOp<8> op;
    fill(op);
    return launch_map(x, y, size, op, as_stream(stream), "pow2_quantize");
  }
  Pow2Op op;
  op.cuts = device_cut_table(kCutPow2Round);
  op.p_max = (float)std::pow(2., e_max);                 // pow2_quantize.cpp:37
  op.p_min = (float)std::pow(2., e_min);                 // :38
  op.thr = (float)((float)op.p_min * std::pow(2., -0.5)); // :39 (float member times double)
  op.e_max = e_max;
  op.e_min = e_min;
  op.sign = sign;
  op.with_zero = with_zero;
  op.lds = nullptr;
  return launch_map(x, y, size, op, as_stream(stream), "pow2_quantize");
}

} // extern "C"

// ---------------------------------------------------------------------- MinMax
namespace nbla_hip {
namespace {

constexpr int kRedBlock = 256;
constexpr int kRedTile = kRedBlock * 4; // elements per block tile
constexpr int kMaxChunks = 1024;

struct MinMaxPlan {
  MinMaxLayout L;
  int64_t tiles_per_row; // tiles covering one run of R1 elements
  int64_t tiles_per_k;   // R0 * tiles_per_row
  int nchunks;           // blocks (and partials) per k
  size_t params_bytes, partial_bytes;
  bool inner;            // the strided pattern takes the kernels of MinMaxInner
  bool rows;             // ... or, its innermost axis reduced (and short runs per channel), those of MinMaxRows
};

MinMaxPlan make_plan(const int64_t *xshape, int ndim, const int64_t *qshape) {
  MinMaxPlan P;
  P.L = collapse(xshape, ndim, qshape);
  P.tiles_per_row = (P.L.R1 + kRedTile - 1) / kRedTile;
  P.tiles_per_k = P.L.R0 * P.tiles_per_row;
  int64_t want = (4096 + P.L.K - 1) / P.L.K;
  if (want > kMaxChunks)
    want = kMaxChunks;
  if (want > P.tiles_per_k)
    want = P.tiles_per_k;
  if (want < 1)
    want = 1;
  P.inner = false;
  if (!P.L.ok || trailing_kept(P.L)) {
    if (!P.L.ok)
      want = 1; // the general strided kernels fold a whole slice per block
    MinMaxAxes A;
    if (split_axes(xshape, ndim, qshape, A)) {
      const MinMaxInner I = inner_form(A);
      if (I.ok) {
        P.inner = true;
        want = inner_chunks(I);
      }
    }
  }
  P.rows = false;
  if (!P.inner && (!P.L.ok || short_rows(P.L))) {
    MinMaxAxes A;
    if (split_axes(xshape, ndim, qshape, A)) {
      const MinMaxRows R = row_form(A);
      if (R.ok) {
        P.rows = true;
        want = row_chunks(R);
      }
    }
  }
  P.nchunks = (int)want;
  P.params_bytes = round_up((size_t)P.L.K * 16, 256);
  P.partial_bytes = round_up((size_t)P.L.K * P.nchunks * 16, 256);
  return P;
}

// min.cpp:29-41 / max.cpp:48-60 scan the slice in index order with strict comparisons starting from +-1e8; of
// several equal extrema the first wins, which is only visible for +0 / -0.  Plain min / max give the value (NaN is
// ignored by both formulations); beside them the first zero of the slice (index and sign) is tracked, and when the
// extremum turns out to be zero it takes that element's sign.  Zeros are rare in most inputs, so their bookkeeping
// sits behind a branch.
struct MinMaxPartial {
  float vmin;
  float vmax;
  uint32_t zidx;  // index of the first +-0 element, 0xffffffff if none
  uint32_t zsign; // its sign bit
};

struct Extrema {
  float vmin, vmax;
  uint32_t zidx, zsign;
  __device__ __forceinline__ void init() {
    vmin = 1e+8f;
    vmax = -1e+8f;
    zidx = 0xffffffffu;
    zsign = 0u;
  }
  __device__ __forceinline__ void take(float v, uint32_t i) { // i increases per thread
    vmin = __builtin_fminf(vmin, v);
    vmax = __builtin_fmaxf(vmax, v);
    const uint32_t u = __float_as_uint(v);
    if ((u << 1) == 0u && zidx == 0xffffffffu) {
      zidx = i;
      zsign = u >> 31;
    }
  }
  __device__ __forceinline__ void take_any(float v, uint32_t i) { // i in any order
    vmin = __builtin_fminf(vmin, v);
    vmax = __builtin_fmaxf(vmax, v);
    const uint32_t u = __float_as_uint(v);
    if ((u << 1) == 0u && i < zidx) {
      zidx = i;
      zsign = u >> 31;
    }
  }
  __device__ __forceinline__ void take4(float4_t v, uint32_t i) {
    vmin = __builtin_fminf(__builtin_fminf(vmin, v.x), __builtin_fminf(v.y, __builtin_fminf(v.z, v.w)));
    vmax = __builtin_fmaxf(__builtin_fmaxf(vmax, v.x), __builtin_fmaxf(v.y, __builtin_fmaxf(v.z, v.w)));
    const uint32_t ux = __float_as_uint(v.x) << 1, uy = __float_as_uint(v.y) << 1;
    const uint32_t uz = __float_as_uint(v.z) << 1, uw = __float_as_uint(v.w) << 1;
    if (min(min(ux, uy), min(uz, uw)) == 0u && zidx == 0xffffffffu) {
      const int c = (ux == 0u) ? 0 : (uy == 0u) ? 1 : (uz == 0u) ? 2 : 3;
      const float z = (c == 0) ? v.x : (c == 1) ? v.y : (c == 2) ? v.z : v.w;
      zidx = i + c;
      zsign = __float_as_uint(z) >> 31;
    }
  }
  __device__ __forceinline__ void merge(float omin, float omax, uint32_t ozidx, uint32_t ozsign) {
    vmin = __builtin_fminf(vmin, omin);
    vmax = __builtin_fmaxf(vmax, omax);
    if (ozidx < zidx) {
      zidx = ozidx;
      zsign = ozsign;
    }
  }
  __device__ __forceinline__ void wave_reduce() {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float a = __shfl_xor(vmin, off);
      const float b = __shfl_xor(vmax, off);
      const uint32_t zi = __shfl_xor(zidx, off);
      const uint32_t zs = __shfl_xor(zsign, off);
      merge(a, b, zi, zs);
    }
  }
  // the extrema as the reference's scan would leave them
  __device__ __forceinline__ float min_value() const {
    return (vmin == 0.0f) ? __uint_as_float(zsign << 31) : vmin;
  }
  __device__ __forceinline__ float max_value() const {
    return (vmax == 0.0f) ? __uint_as_float(zsign << 31) : vmax;
  }
  __device__ __forceinline__ MinMaxPartial pack() const { return MinMaxPartial{vmin, vmax, zidx, zsign}; }
};

// Stage 1: block (chunk c, channel k) scans tiles c, c+nchunks, ... of channel k.
template <bool kVec>
__global__ __launch_bounds__(kRedBlock) void minmax_reduce_tiles(const float *__restrict__ x, MinMaxPartial *__restrict__ partial,
                                                                 int64_t K, int64_t R1, int64_t tiles_per_row,
                                                                 int64_t tiles_per_k, int nchunks) {
  const int64_t k = blockIdx.y;
  Extrema ex;
  ex.init();
  for (int64_t t = blockIdx.x; t < tiles_per_k; t += nchunks) {
    const int64_t r0 = t / tiles_per_row;
    const int64_t r1 = (t - r0 * tiles_per_row) * kRedTile + 4 * threadIdx.x;
    if (r1 >= R1)
      continue;
    const float *p = x + (r0 * K + k) * R1 + r1;
    const uint32_t idx = (uint32_t)(r0 * R1 + r1);
    if (kVec) { // R1 % 4 == 0 and x 16-byte aligned
      const float4_t v = *reinterpret_cast<const float4_t *>(p);
      ex.take4(v, idx);
    } else {
      const int n = (R1 - r1) < 4 ? (int)(R1 - r1) : 4;
      for (int j = 0; j < n; ++j)
        ex.take(p[j], idx + j);
    }
  }
  ex.wave_reduce();
  __shared__ MinMaxPartial s_part[kRedBlock / 64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0)
    s_part[wave] = ex.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRedBlock / 64; ++w)
      ex.merge(s_part[w].vmin, s_part[w].vmax, s_part[w].zidx, s_part[w].zsign);
    partial[k * nchunks + blockIdx.x] = ex.pack();
  }
}

// Per-tensor stage 1 (K == 1, 16-byte aligned): every block scans one contiguous range.
__global__ __launch_bounds__(kRedBlock) void minmax_reduce_flat(const float *__restrict__ x, MinMaxPartial *__restrict__ partial,
                                                                size_t n4, size_t size) {
  Extrema ex;
  ex.init();
  // block b streams the contiguous range [b * per, (b + 1) * per) of float4s, four 128-bit loads in flight per thread
  const size_t per = (n4 + gridDim.x - 1) / gridDim.x;
  const size_t begin = (size_t)blockIdx.x * per, end = (begin + per < n4) ? begin + per : n4;
  size_t i = begin + threadIdx.x;
  for (; i + 3 * kRedBlock < end; i += 4 * kRedBlock) {
    float4_t v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      v[j] = load4(x + 4 * (i + j * kRedBlock));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t idx = (uint32_t)(4 * (i + j * kRedBlock));
      ex.take4(v[j], idx);
    }
  }
  for (; i < end; i += kRedBlock) {
    const float4_t v = load4(x + 4 * i);
    const uint32_t idx = (uint32_t)(4 * i);
    ex.take4(v, idx);
  }
  if (blockIdx.x == gridDim.x - 1) { // tail elements, highest indices
    const size_t t = 4 * n4 + threadIdx.x;
    if (t < size)
      ex.take(x[t], (uint32_t)t);
  }
  ex.wave_reduce();
  __shared__ MinMaxPartial s_part[kRedBlock / 64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0)
    s_part[wave] = ex.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRedBlock / 64; ++w)
      ex.merge(s_part[w].vmin, s_part[w].vmax, s_part[w].zidx, s_part[w].zsign);
    partial[blockIdx.x] = ex.pack();
  }
}

// Stage 2: one wavefront per channel folds the partials, then lane 0 applies the
// EMA (min_max_quantize.cpp:159-178), nudge_range (:353-361), the scale
// (:188-190) and nudge_qr_min_max (:363-390), one rounded fp32 op at a time.
struct MinMaxScalars {
  float decay, one_minus_decay, eps;
  int x_min_max, ema;
};

// The nudged range, scale and zero point of one range from its extrema (min_max_quantize.cpp:130-211), every
// operation rounded on its own.
__device__ __forceinline__ void minmax_finalize_range(const Extrema &ex, int64_t k, float *__restrict__ qr_min,
                                                      float *__restrict__ qr_max, const float *__restrict__ ql_min,
                                                      const float *__restrict__ ql_max, float *__restrict__ scale_out,
                                                      float4_t *__restrict__ params, const MinMaxScalars &s) {
  float lo = qr_min[k], hi = qr_max[k];
  if (s.x_min_max && s.ema) {
    const float a = ex.min_value() * s.one_minus_decay;
    lo = lo * s.decay;
    lo = lo + a;
    const float b = ex.max_value() * s.one_minus_decay;
    hi = hi * s.decay;
    hi = hi + b;
  } else if (s.x_min_max) {
    lo = ex.min_value();
    hi = ex.max_value();
  }
  if (hi - lo < s.eps)
    hi = lo + s.eps;
  qr_min[k] = lo;
  qr_max[k] = hi;
  const float qlo = ql_min[k], qhi = ql_max[k];
  float scale = hi - lo;
  const float levels = qhi - qlo;
  scale = scale / levels;
  const float zp_from_min = qlo - lo / scale;
  float zp;
  if (zp_from_min <= qlo)
    zp = qlo;
  else if (zp_from_min >= qhi)
    zp = qhi;
  else
    zp = round_half_away(zp_from_min);
  const float m_n = (qlo - zp) * scale;
  const float M_n = (qhi - zp) * scale;
  scale_out[k] = scale;
  float4_t pr;
  pr.x = m_n;
  pr.y = M_n;
  pr.z = scale;
  pr.w = 0.0f;
  params[k] = pr;
}

__global__ __launch_bounds__(64) void minmax_finalize(const MinMaxPartial *__restrict__ partial, int nchunks,
                                                      float *__restrict__ qr_min, float *__restrict__ qr_max,
                                                      const float *__restrict__ ql_min,
                                                      const float *__restrict__ ql_max, float *__restrict__ scale_out,
                                                      float4_t *__restrict__ params, MinMaxScalars s) {
  const int64_t k = blockIdx.x;
  Extrema ex;
  ex.init();
  if (s.x_min_max) {
    // sixteen independent 16-byte loads in flight per lane before any merge: one round trip for 1024 partials
    const float4_t *pp = reinterpret_cast<const float4_t *>(partial + k * nchunks);
    for (int c = threadIdx.x; c < nchunks; c += 1024) {
      float4_t q[16];
#pragma unroll
      for (int j = 0; j < 16; ++j)
        q[j] = (c + 64 * j < nchunks) ? pp[c + 64 * j] : float4_t{1e+8f, -1e+8f, __uint_as_float(0xffffffffu), 0.0f};
#pragma unroll
      for (int j = 0; j < 16; ++j)
        ex.merge(q[j].x, q[j].y, __float_as_uint(q[j].z), __float_as_uint(q[j].w));
    }
    ex.wave_reduce();
  }
  if (threadIdx.x != 0)
    return;
  minmax_finalize_range(ex, k, qr_min, qr_max, ql_min, ql_max, scale_out, params, s);
}

// Many ranges of few partial results each (ranges per channel and column, say): a thread per range instead of a
// wavefront per range.  The merge does not depend on the order (extrema, and the first zero by its index).
__global__ __launch_bounds__(256) void minmax_finalize_many(const MinMaxPartial *__restrict__ partial, int nchunks,
                                                            int64_t K, float *__restrict__ qr_min,
                                                            float *__restrict__ qr_max,
                                                            const float *__restrict__ ql_min,
                                                            const float *__restrict__ ql_max,
                                                            float *__restrict__ scale_out,
                                                            float4_t *__restrict__ params, MinMaxScalars s) {
  const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (k >= K)
    return;
  Extrema ex;
  ex.init();
  if (s.x_min_max) {
    const float4_t *pp = reinterpret_cast<const float4_t *>(partial + k * nchunks);
    for (int c = 0; c < nchunks; ++c) {
      const float4_t q = pp[c];
      ex.merge(q.x, q.y, __float_as_uint(q.z), __float_as_uint(q.w));
    }
  }
  minmax_finalize_range(ex, k, qr_min, qr_max, ql_min, ql_max, scale_out, params, s);
}

// One wavefront per range, or one thread per range where the ranges are many and their partial results few.
void launch_minmax_finalize(int64_t K, const MinMaxPartial *partial, int nchunks, float *qr_min, float *qr_max,
                            const float *ql_min, const float *ql_max, float *scale, float4_t *params,
                            const MinMaxScalars &sc, hipStream_t stream) {
  if (K >= 256 && nchunks <= 16)
    hipLaunchKernelGGL(minmax_finalize_many, dim3((unsigned)((K + 255) / 256)), dim3(256), 0, stream, partial, nchunks, K,
                       qr_min, qr_max, ql_min, ql_max, scale, params, sc);
  else
    hipLaunchKernelGGL(minmax_finalize, dim3((unsigned)K), dim3(64), 0, stream, partial, nchunks, qr_min, qr_max, ql_min,
                       ql_max, scale, params, sc);
}

// min_max_quantize.cpp:213-222: seven separately rounded fp32 operations.
__device__ __forceinline__ float minmax_apply(float x, float m_n, float M_n, float scale) {
  float t = (x > m_n) ? x : m_n;
  t = (t < M_n) ? t : M_n;
  t = t - m_n;
  t = t / scale;
  t = round_half_away(t);
  t = t * scale;
  return t + m_n;
}

// Stage 3a: per-tensor, 16-byte aligned.
__global__ __launch_bounds__(kBlock) void minmax_apply_flat(const float *__restrict__ x, float *__restrict__ y, size_t n4,
                                                            size_t size, const float4_t *__restrict__ params) {
  const float4_t pr = params[0];
  const size_t base = (size_t)blockIdx.x * kTile + threadIdx.x;
  float4_t v[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4)
      v[j] = load4(x + 4 * i);
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const size_t i = base + (size_t)j * kBlock;
    if (i < n4) {
      float4_t r;
      r.x = minmax_apply(v[j].x, pr.x, pr.y, pr.z);
      r.y = minmax_apply(v[j].y, pr.x, pr.y, pr.z);
      r.z = minmax_apply(v[j].z, pr.x, pr.y, pr.z);
      r.w = minmax_apply(v[j].w, pr.x, pr.y, pr.z);
      store4(y + 4 * i, r);
    }
  }
  if (blockIdx.x == 0) {
    const size_t i = 4 * n4 + threadIdx.x;
    if (i < size)
      y[i] = minmax_apply(x[i], pr.x, pr.y, pr.z);
  }
}

// Stage 3b: per-channel rows of R1 contiguous elements (R1 % 4 == 0, aligned):
// blockIdx.x = row (r0 * K + k), blockIdx.y = tile along the row.
__global__ __launch_bounds__(kBlock) void minmax_apply_rows(const float *__restrict__ x, float *__restrict__ y, int64_t K,
                                                            int64_t R1, const float4_t *__restrict__ params) {
  const int64_t row = blockIdx.x;
  const float4_t pr = params[row % K];
  const int64_t n4 = R1 / 4;
  const float *xr = x + row * R1;
  float *yr = y + row * R1;
  for (int64_t i = (int64_t)blockIdx.y * kBlock + threadIdx.x; i < n4; i += (int64_t)gridDim.y * kBlock) {
    const float4_t v = load4(xr + 4 * i);
    float4_t r;
    r.x = minmax_apply(v.x, pr.x, pr.y, pr.z);
    r.y = minmax_apply(v.y, pr.x, pr.y, pr.z);
    r.z = minmax_apply(v.z, pr.x, pr.y, pr.z);
    r.w = minmax_apply(v.w, pr.x, pr.y, pr.z);
    store4(yr + 4 * i, r);
  }
}

// Stage 3c: any layout / alignment, one element per step.
__global__ __launch_bounds__(kBlock) void minmax_apply_generic(const float *__restrict__ x, float *__restrict__ y, int64_t total,
                                                               int64_t K, int64_t R1,
                                                               const float4_t *__restrict__ params) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
    const float4_t pr = params[(i / R1) % K];
    y[i] = minmax_apply(x[i], pr.x, pr.y, pr.z);
  }
}


// Any pattern of kept and reduced axes (e.g. q shape (C, 1, W)): block k scans the slice of kept index k in the order
// the reference's Min / Max scan it (reduced axes row-major), one element per thread and step.
__global__ __launch_bounds__(kRedBlock) void minmax_reduce_strided(const float *__restrict__ x,
                                                                   MinMaxPartial *__restrict__ partial, MinMaxAxes A,
                                                                   int64_t R) {
  const int64_t k = blockIdx.x;
  const float *base = x + strided_offset(k, A.nkept, A.ksize, A.kstride);
  Extrema ex;
  ex.init();
  for (int64_t r = threadIdx.x; r < R; r += kRedBlock)
    ex.take(base[strided_offset(r, A.nred, A.rsize, A.rstride)], (uint32_t)r);
  ex.wave_reduce();
  __shared__ MinMaxPartial s_part[kRedBlock / 64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0)
    s_part[wave] = ex.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRedBlock / 64; ++w)
      ex.merge(s_part[w].vmin, s_part[w].vmax, s_part[w].zidx, s_part[w].zsign);
    partial[k] = ex.pack();
  }
}
template <int kVec>
__global__ __launch_bounds__(kRedBlock) void minmax_reduce_inner(const float *__restrict__ x,
                                                                 MinMaxPartial *__restrict__ partial, MinMaxAxes A,
                                                                 MinMaxInner I, int nchunks) {
  __shared__ MinMaxPartial s_part[kRedBlock / 64][64][kVec];
  const int64_t ko = blockIdx.x;
  const int chunk = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tw = I.tw, rows_per_step = kRedBlock / tw;
  const int cw = tid & (tw - 1), slot = tid / tw; // column (quad) inside the pass, row slot inside the step
  const InnerWalk W = inner_walk(x, A, I, ko, chunk, nchunks);
  constexpr int kRows = kVec == 4 ? 4 : 8; // rows in flight per lane
  for (int64_t w0 = 0; w0 < I.Wk; w0 += (int64_t)tw * kVec) {
    const int64_t wcol = w0 + (int64_t)cw * kVec;
    const bool col_in = wcol < I.Wk;
    Extrema ex[kVec];
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      ex[c].init();
    for (int64_t ro = W.ro_begin; ro < W.ro_end; ++ro) {
      const float *row0 = W.base + (A.nred > 1 ? strided_offset(ro, A.nred - 1, A.rsize, A.rstride) : 0) + wcol;
      for (int64_t ri0 = 0; ri0 < I.Rin; ri0 += kRows * rows_per_step) {
        InnerRow<kVec> v[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          if (col_in && ri < I.Rin)
            v[j].load(row0 + ri * I.rin_stride);
          else
            v[j].fill(__uint_as_float(0x7fc00000u)); // NaN: ignored by the scan
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
#pragma unroll
          for (int c = 0; c < kVec; ++c)
            ex[c].take(v[j].v[c], (uint32_t)(ro * I.Rin + ri));
        }
      }
    }
    // fold the row slots that share a column: across the lanes of a wavefront, then across the wavefronts
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      for (int off = 32; off >= tw; off >>= 1) {
        const float a = __shfl_xor(ex[c].vmin, off), b = __shfl_xor(ex[c].vmax, off);
        const uint32_t zi = __shfl_xor(ex[c].zidx, off), zs = __shfl_xor(ex[c].zsign, off);
        ex[c].merge(a, b, zi, zs);
      }
    __syncthreads(); // the previous pass's partial results have been read
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      s_part[wave][lane][c] = ex[c].pack();
    __syncthreads();
    if (tid < tw && col_in) {
#pragma unroll
      for (int c = 0; c < kVec; ++c) {
        Extrema all;
        all.init();
        for (int w = 0; w < kRedBlock / 64; ++w)
          all.merge(s_part[w][tid][c].vmin, s_part[w][tid][c].vmax, s_part[w][tid][c].zidx, s_part[w][tid][c].zsign);
        partial[(ko * I.Wk + wcol + c) * nchunks + chunk] = all.pack();
      }
    }
  }
}
template <int kVec>
__global__ __launch_bounds__(kRedBlock) void minmax_apply_inner(const float *__restrict__ x, float *__restrict__ y,
                                                                MinMaxAxes A, MinMaxInner I, int nchunks,
                                                                const float4_t *__restrict__ params) {
  const int64_t ko = blockIdx.x;
  const int chunk = blockIdx.y, tid = threadIdx.x;
  const int tw = I.tw, rows_per_step = kRedBlock / tw;
  const int cw = tid & (tw - 1), slot = tid / tw;
  const InnerWalk W = inner_walk(x, A, I, ko, chunk, nchunks);
  constexpr int kRows = kVec == 4 ? 4 : 8;
  for (int64_t w0 = 0; w0 < I.Wk; w0 += (int64_t)tw * kVec) {
    const int64_t wcol = w0 + (int64_t)cw * kVec;
    const bool col_in = wcol < I.Wk;
    float4_t pr[kVec];
#pragma unroll
    for (int c = 0; c < kVec; ++c)
      pr[c] = params[ko * I.Wk + (col_in ? wcol + c : 0)];
    for (int64_t ro = W.ro_begin; ro < W.ro_end; ++ro) {
      const int64_t off = (W.base - x) + (A.nred > 1 ? strided_offset(ro, A.nred - 1, A.rsize, A.rstride) : 0) + wcol;
      for (int64_t ri0 = 0; ri0 < I.Rin; ri0 += kRows * rows_per_step) {
        InnerRow<kVec> v[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          if (col_in && ri < I.Rin)
            v[j].load(x + off + ri * I.rin_stride);
          else
            v[j].fill(0.0f);
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          if (col_in && ri < I.Rin) {
            float *dst = y + off + ri * I.rin_stride;
            if (kVec == 4) {
              float4_t r;
              r.x = minmax_apply(v[j].v[0], pr[0].x, pr[0].y, pr[0].z);
              r.y = minmax_apply(v[j].v[1 % kVec], pr[1 % kVec].x, pr[1 % kVec].y, pr[1 % kVec].z);
              r.z = minmax_apply(v[j].v[2 % kVec], pr[2 % kVec].x, pr[2 % kVec].y, pr[2 % kVec].z);
              r.w = minmax_apply(v[j].v[3 % kVec], pr[3 % kVec].x, pr[3 % kVec].y, pr[3 % kVec].z);
              __builtin_nontemporal_store(r, reinterpret_cast<float4_t *>(dst));
            } else {
              __builtin_nontemporal_store(minmax_apply(v[j].v[0], pr[0].x, pr[0].y, pr[0].z), dst);
            }
          }
        }
      }
    }
  }
}
// The row form (MinMaxRows: the innermost axis reduced, T lanes per run).  Block (tile of 256 / T kept indices,
// chunk); a thread's elements all belong to its kept index, so it keeps one set of extrema, which the T lanes of the
// run then fold.
template <int kVec>
__global__ __launch_bounds__(kRedBlock) void minmax_reduce_rowform(const float *__restrict__ x,
                                                                   MinMaxPartial *__restrict__ partial, MinMaxAxes A,
                                                                   MinMaxRows R, int T, int nchunks) {
  const int tid = threadIdx.x, li = tid & (T - 1), slot = tid / T, rps = kRedBlock / T;
  const int64_t k = (int64_t)blockIdx.x * rps + slot;
  const bool k_in = k < R.K;
  const int chunk = blockIdx.y;
  const RowWalk W = row_walk(R, chunk, nchunks);
  const float *base = x + strided_offset(k_in ? k : 0, A.nkept, A.ksize, A.kstride);
  Extrema ex;
  ex.init();
  constexpr int kRows = 4; // outer reduced indices in flight per lane
  for (int64_t ro = W.ro_begin; ro < W.ro_end; ro += kRows) {
    int64_t off[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j)
      off[j] = (A.nred > 1 && ro + j < W.ro_end) ? strided_offset(ro + j, A.nred - 1, A.rsize, A.rstride) : 0;
    for (int64_t ri0 = 0; ri0 < R.Rin; ri0 += (int64_t)T * kVec) {
      const int64_t ri = ri0 + (int64_t)li * kVec;
      InnerRow<kVec> v[kRows];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (k_in && ro + j < W.ro_end && ri < R.Rin)
          v[j].load(base + off[j] + ri);
        else
          v[j].fill(__uint_as_float(0x7fc00000u)); // NaN: ignored by the scan
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j)
#pragma unroll
        for (int c = 0; c < kVec; ++c)
          ex.take_any(v[j].v[c], (uint32_t)((ro + j) * R.Rin + ri + c));
    }
  }
  for (int o = T >> 1; o >= 1; o >>= 1) {
    const float a = __shfl_xor(ex.vmin, o), b = __shfl_xor(ex.vmax, o);
    const uint32_t zi = __shfl_xor(ex.zidx, o), zs = __shfl_xor(ex.zsign, o);
    ex.merge(a, b, zi, zs);
  }
  if (li == 0 && k_in)
    partial[k * nchunks + chunk] = ex.pack();
}
template <int kVec>
__global__ __launch_bounds__(kRedBlock) void minmax_apply_rowform(const float *__restrict__ x, float *__restrict__ y,
                                                                  MinMaxAxes A, MinMaxRows R, int T, int nchunks,
                                                                  const float4_t *__restrict__ params) {
  const int tid = threadIdx.x, li = tid & (T - 1), slot = tid / T, rps = kRedBlock / T;
  const int64_t k = (int64_t)blockIdx.x * rps + slot;
  const bool k_in = k < R.K;
  const int chunk = blockIdx.y;
  const RowWalk W = row_walk(R, chunk, nchunks);
  const int64_t base = strided_offset(k_in ? k : 0, A.nkept, A.ksize, A.kstride);
  const float4_t pr = params[k_in ? k : 0];
  constexpr int kRows = 4;
  for (int64_t ro = W.ro_begin; ro < W.ro_end; ro += kRows) {
    int64_t off[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j)
      off[j] = base + ((A.nred > 1 && ro + j < W.ro_end) ? strided_offset(ro + j, A.nred - 1, A.rsize, A.rstride) : 0);
    for (int64_t ri0 = 0; ri0 < R.Rin; ri0 += (int64_t)T * kVec) {
      const int64_t ri = ri0 + (int64_t)li * kVec;
      InnerRow<kVec> v[kRows];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (k_in && ro + j < W.ro_end && ri < R.Rin)
          v[j].load(x + off[j] + ri);
        else
          v[j].fill(0.0f);
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (!(k_in && ro + j < W.ro_end && ri < R.Rin))
          continue;
        float *dst = y + off[j] + ri;
        if (kVec == 4) {
          float4_t r;
          r.x = minmax_apply(v[j].v[0], pr.x, pr.y, pr.z);
          r.y = minmax_apply(v[j].v[1 % kVec], pr.x, pr.y, pr.z);
          r.z = minmax_apply(v[j].v[2 % kVec], pr.x, pr.y, pr.z);
          r.w = minmax_apply(v[j].v[3 % kVec], pr.x, pr.y, pr.z);
          __builtin_nontemporal_store(r, reinterpret_cast<float4_t *>(dst));
        } else {
          __builtin_nontemporal_store(minmax_apply(v[j].v[0], pr.x, pr.y, pr.z), dst);
        }
      }
    }
  }
}
// Element i of x (dense, row-major) belongs to the kept index formed by its coordinates along the kept axes.
__global__ __launch_bounds__(kBlock) void minmax_apply_strided(const float *__restrict__ x, float *__restrict__ y,
                                                               int64_t total, MinMaxAxes A,
                                                               const float4_t *__restrict__ params) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
    int64_t k = 0;
    for (int d = 0; d < A.nkept; ++d)
      k = k * A.ksize[d] + (i / A.kstride[d]) % A.ksize[d];
    const float4_t pr = params[k];
    y[i] = minmax_apply(x[i], pr.x, pr.y, pr.z);
  }
}

// The whole forward on caller-provided scratch (`workspace`: the nudged-range table, then the reduction partials).
// Every word of the scratch that a launch reads has been written earlier in the same call, so nothing has to start
// at zero.  `scratch_limit` != 0 marks the fixed-size scratch of the allocation-free entry point.
int min_max_quantize_forward(const float *x, float *y, const int64_t *xshape, int ndim, const int64_t *qshape,
                             float *qr_min, float *qr_max, const float *ql_min, const float *ql_max, float *scale,
                             float decay, int x_min_max, int ema, float eps, void *workspace, size_t workspace_bytes,
                             size_t scratch_limit, void *stream_) {
  for (int i = 0; i < ndim; ++i)
    if (qshape[i] != 1 && qshape[i] != xshape[i])
      return fail(NBLA_HIP_ERR_VALUE,
                  "x.shape and ql_min.shape must be same except for i-th dimension where ql_min.shape[i] == 1.");
  MinMaxPlan P = make_plan(xshape, ndim, qshape);
  MinMaxAxes axes;
  if ((!P.L.ok || P.inner || P.rows) && !split_axes(xshape, ndim, qshape, axes))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "more than eight kept or eight reduced axes of size above one.");
  if (P.L.total == 0)
    return NBLA_HIP_OK;
  if (scratch_limit && (P.inner || P.rows) && P.params_bytes + P.partial_bytes > scratch_limit) {
    P.nchunks = 1; // the fixed scratch holds one partial result per range
    P.partial_bytes = round_up((size_t)P.L.K * 16, 256);
  }
  if (P.L.R0 * P.L.R1 > 0xffffffffll)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "reduction slices above 2^32 elements are not supported.");
  if (scratch_limit && P.params_bytes + P.partial_bytes > scratch_limit)
    return fail(NBLA_HIP_ERR_MEMORY,
                "min_max_quantize: %lld quantization ranges need %zu bytes of scratch, above the %zu bytes of the "
                "allocation-free entry point; use nbla_hip_min_max_quantize_f32 with a workspace.",
                (long long)P.L.K, P.params_bytes + P.partial_bytes, scratch_limit);
  if (workspace_bytes < P.params_bytes + P.partial_bytes || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "min_max_quantize workspace too small or misaligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  float4_t *params = static_cast<float4_t *>(workspace);
  MinMaxPartial *partial = reinterpret_cast<MinMaxPartial *>(static_cast<char *>(workspace) + P.params_bytes);
  const MinMaxLayout &L = P.L;
  const bool vec_ok = aligned16(x) && (L.R1 % 4 == 0 || L.K == 1);
  int nchunks = P.nchunks;

  if (!L.ok || P.inner || P.rows) { // kept axes separated by reduced ones, all behind them, or short runs
    if (L.K > 0x7fffffffll)
      return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "more than 2^31 - 1 quantization ranges.");
    MinMaxInner inner = P.inner ? inner_form(axes) : MinMaxInner{false};
    if (inner.ok) {
      // four columns per lane where the rows allow 128-bit accesses (every other stride is a multiple of Wk)
      const bool quads = inner.Wk % 4 == 0 && aligned16(x) && aligned16(y);
      if (quads) {
        inner.tw = 1;
        while (inner.tw < 64 && inner.tw * 4 < inner.Wk)
          inner.tw *= 2;
      }
      const dim3 grid((unsigned)inner.Ko, (unsigned)nchunks);
      if (x_min_max) {
        if (quads)
          hipLaunchKernelGGL(minmax_reduce_inner<4>, grid, dim3(kRedBlock), 0, stream, x, partial, axes, inner, nchunks);
        else
          hipLaunchKernelGGL(minmax_reduce_inner<1>, grid, dim3(kRedBlock), 0, stream, x, partial, axes, inner, nchunks);
        NBLA_HIP_LAUNCH_CHECK("min_max_quantize reduction");
      }
      MinMaxScalars sc;
      sc.decay = (float)decay;
      sc.one_minus_decay = (float)(1.0 - (double)decay);
      sc.eps = eps;
      sc.x_min_max = x_min_max;
      sc.ema = ema;
      launch_minmax_finalize(L.K, partial, nchunks, qr_min, qr_max, ql_min, ql_max, scale, params, sc, stream);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize finalize");
      if (quads)
        hipLaunchKernelGGL(minmax_apply_inner<4>, grid, dim3(kRedBlock), 0, stream, x, y, axes, inner, nchunks, params);
      else
        hipLaunchKernelGGL(minmax_apply_inner<1>, grid, dim3(kRedBlock), 0, stream, x, y, axes, inner, nchunks, params);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize apply");
      return NBLA_HIP_OK;
    }
    if (P.rows) {
      const MinMaxRows R = row_form(axes);
      const bool quads = R.Rin % 4 == 0 && aligned16(x) && aligned16(y);
      const int T = row_lanes(R, quads ? 4 : 1);
      const int64_t rps = kRedBlock / T;
      const dim3 grid((unsigned)((R.K + rps - 1) / rps), (unsigned)nchunks);
      if (x_min_max) {
        if (quads)
          hipLaunchKernelGGL(minmax_reduce_rowform<4>, grid, dim3(kRedBlock), 0, stream, x, partial, axes, R, T, nchunks);
        else
          hipLaunchKernelGGL(minmax_reduce_rowform<1>, grid, dim3(kRedBlock), 0, stream, x, partial, axes, R, T, nchunks);
        NBLA_HIP_LAUNCH_CHECK("min_max_quantize reduction");
      }
      MinMaxScalars sc;
      sc.decay = (float)decay;
      sc.one_minus_decay = (float)(1.0 - (double)decay);
      sc.eps = eps;
      sc.x_min_max = x_min_max;
      sc.ema = ema;
      launch_minmax_finalize(L.K, partial, nchunks, qr_min, qr_max, ql_min, ql_max, scale, params, sc, stream);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize finalize");
      if (quads)
        hipLaunchKernelGGL(minmax_apply_rowform<4>, grid, dim3(kRedBlock), 0, stream, x, y, axes, R, T, nchunks, params);
      else
        hipLaunchKernelGGL(minmax_apply_rowform<1>, grid, dim3(kRedBlock), 0, stream, x, y, axes, R, T, nchunks, params);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize apply");
      return NBLA_HIP_OK;
    }
    if (x_min_max) {
      hipLaunchKernelGGL(minmax_reduce_strided, dim3((unsigned)L.K), dim3(kRedBlock), 0, stream, x, partial, axes,
                         L.R1);
      NBLA_HIP_LAUNCH_CHECK("min_max_quantize reduction");
    }
    MinMaxScalars sc;
    sc.decay = (float)decay;
    sc.one_minus_decay = (float)(1.0 - (double)decay);
    sc.eps = eps;
    sc.x_min_max = x_min_max;
    sc.ema = ema;
    launch_minmax_finalize(L.K, partial, 1, qr_min, qr_max, ql_min, ql_max, scale, params, sc, stream);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize finalize");
    int64_t blocks = (L.total + kBlock - 1) / kBlock;
    if (blocks > 65536)
      blocks = 65536;
    hipLaunchKernelGGL(minmax_apply_strided, dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, L.total, axes,
                       params);
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize apply");
    return NBLA_HIP_OK;
  }

  if (x_min_max) {
    if (L.K == 1 && aligned16(x)) {
      const size_t n4 = (size_t)L.total / 4;
      size_t blocks = (n4 + kRedBlock * 4 - 1) / (kRedBlock * 4);
      if (blocks > (size_t)nchunks)
        blocks = nchunks;
      if (blocks < 1)
        blocks = 1;
      nchunks = (int)blocks;
      hipLaunchKernelGGL(minmax_reduce_flat, dim3((unsigned)blocks), dim3(kRedBlock), 0, stream, x, partial, n4,
                         (size_t)L.total);
    } else if (vec_ok && L.R1 % 4 == 0) {
      hipLaunchKernelGGL(minmax_reduce_tiles<true>, dim3(nchunks, (unsigned)L.K), dim3(kRedBlock), 0, stream, x,
                         partial, L.K, L.R1, P.tiles_per_row, P.tiles_per_k, nchunks);
    } else {
      hipLaunchKernelGGL(minmax_reduce_tiles<false>, dim3(nchunks, (unsigned)L.K), dim3(kRedBlock), 0, stream, x,
                         partial, L.K, L.R1, P.tiles_per_row, P.tiles_per_k, nchunks);
    }
    NBLA_HIP_LAUNCH_CHECK("min_max_quantize reduction");
  }
  MinMaxScalars s;
  s.decay = (float)decay;                            // (T)(decay_)        min_max_quantize.cpp:105
  s.one_minus_decay = (float)(1.0 - (double)decay);  // (T)(1.0 - decay_)  :106
  s.eps = eps;
  s.x_min_max = x_min_max;
  s.ema = ema;
  launch_minmax_finalize(L.K, partial, nchunks, qr_min, qr_max, ql_min, ql_max, scale, params, s, stream);
  NBLA_HIP_LAUNCH_CHECK("min_max_quantize finalize");

  if (L.K == 1 && aligned16(x) && aligned16(y)) {
    const size_t n4 = (size_t)L.total / 4;
    const size_t blocks = n4 ? (n4 + kTile - 1) / kTile : 1;
    hipLaunchKernelGGL(minmax_apply_flat, dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, n4, (size_t)L.total,
                       params);
  } else if (aligned16(x) && aligned16(y) && L.R1 % 4 == 0 && L.R1 >= 256 && L.R0 * L.K < 0x7fffffffll) {
    int64_t ytiles = (L.R1 / 4 + kBlock - 1) / kBlock;
    if (ytiles > 64)
      ytiles = 64;
    hipLaunchKernelGGL(minmax_apply_rows, dim3((unsigned)(L.R0 * L.K), (unsigned)ytiles), dim3(kBlock), 0, stream, x,
                       y, L.K, L.R1, params);
  } else {
    int64_t blocks = (L.total + kBlock - 1) / kBlock;
    if (blocks > 65536)
      blocks = 65536;
    hipLaunchKernelGGL(minmax_apply_generic, dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, y, L.total, L.K, L.R1,
                       params);
  }
  NBLA_HIP_LAUNCH_CHECK("min_max_quantize apply");
  return NBLA_HIP_OK;
}

// ---- scratch of the allocation-free entry point: one copy per device that loads this library, held until the
// process ends.  Host code never uses the array's name as an address: the per-device address comes from
// hipGetSymbolAddress, once per device, and is what the kernels receive.
constexpr size_t kStaticScratchBytes = NBLA_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxScratchDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<void *> g_scratch_ptr[kMaxScratchDevices] = {};

} // namespace

int register_static_scratch(int device) {
  if (device < 0 || device >= kMaxScratchDevices)
    return fail(NBLA_HIP_ERR_VALUE, "device index %d out of range", device);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device].load(std::memory_order_acquire))
    return NBLA_HIP_OK;
  int current = -1;
  hipError_t e = hipGetDevice(&current);
  if (e != hipSuccess)
    return fail_hip(e, "hipGetDevice");
  if (current != device)
    return fail(NBLA_HIP_ERR_RUNTIME, "static scratch of device %d asked for while device %d is current", device,
                current);
  void *ptr = nullptr;
  e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess)
    return fail_hip(e, "hipGetSymbolAddress(static scratch)");
  if (!ptr || !aligned256(ptr))
    return fail(NBLA_HIP_ERR_RUNTIME, "static scratch of device %d resolved to a null or misaligned address", device);
  g_scratch_ptr[device].store(ptr, std::memory_order_release);
  return NBLA_HIP_OK;
}

} // namespace nbla_hip

extern "C" {

size_t nbla_hip_min_max_quantize_workspace_bytes(const int64_t *xshape, int ndim, const int64_t *qshape) {
  const MinMaxPlan P = make_plan(xshape, ndim, qshape);
  return P.params_bytes + P.partial_bytes;
}

int nbla_hip_min_max_quantize_f32(const float *x, float *y, const int64_t *xshape, int ndim, const int64_t *qshape,
                                  float *qr_min, float *qr_max, const float *ql_min, const float *ql_max, float *scale,
                                  float decay, int x_min_max, int ema, float eps, void *workspace,
                                  size_t workspace_bytes, void *stream_) {
  return min_max_quantize_forward(x, y, xshape, ndim, qshape, qr_min, qr_max, ql_min, ql_max, scale, decay, x_min_max,
                                  ema, eps, workspace, workspace_bytes, 0, stream_);
}

int nbla_hip_min_max_quantize_static_f32(const float *x, float *y, const int64_t *xshape, int ndim,
                                         const int64_t *qshape, float *qr_min, float *qr_max, const float *ql_min,
                                         const float *ql_max, float *scale, float decay, int x_min_max, int ema,
                                         float eps, void *stream_) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail_hip(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxScratchDevices)
    return fail(NBLA_HIP_ERR_VALUE, "device index %d out of range", dev);
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr)
    return fail(NBLA_HIP_ERR_RUNTIME,
                "nbla_hip_min_max_quantize_static_f32: call nbla_hip_init(%d) first (it resolves the device's "
                "scratch address; this entry point does no set-up of its own).", dev);
  return min_max_quantize_forward(x, y, xshape, ndim, qshape, qr_min, qr_max, ql_min, ql_max, scale, decay, x_min_max,
                                  ema, eps, ptr, kStaticScratchBytes, kStaticScratchBytes, stream_);
}

} // extern "C"

// ------------------------------------------------------------------ range recorders
// The recorders of quantization-aware training (python/src/nnabla/utils/qnn.py:42-560) are identity functions that
// keep running statistics of what passes through them: y = x, and while training the one-element arrays m / M take
//   kMinMaxMinMax  m = minimum2(m, min x), M = maximum2(M, max x)                     (qnn.py:73-84)
//   kAbsMax        M = maximum2(M, max |x|)                                           (qnn.py:178-188)
//   kMinMaxMva     m = decay * m + (1 - decay) * min x, M likewise with max x         (qnn.py:289-300)
//   kMaxMax        M = maximum2(M, max x)                                             (qnn.py:411-420)
//   kMaxMva        M = decay * M + (1 - decay) * max x                                (qnn.py:509-518)
// with min / max as max.cpp / min.cpp compute them (see Extrema above).  One pass copies x to y and scans it.
namespace nbla_hip {
namespace {

enum RecorderMode { kMinMaxMinMax = 0, kAbsMax = 1, kMinMaxMva = 2, kMaxMax = 3, kMaxMva = 4, kRecorderModes = 5 };

// The statistic's update from the extrema of the whole array: what runs after the scan.
__device__ __forceinline__ void record_apply(const Extrema &ex, float *__restrict__ m, float *__restrict__ M, int mode,
                                             float decay, float one_minus_decay) {
  const float mb = ex.min_value(), Mb = ex.max_value();
  if (mode == kMinMaxMinMax) {
    const float lo = *m, hi = *M;
    *m = (lo < mb) ? lo : mb; // minimum2.hpp:41
    *M = (hi > Mb) ? hi : Mb; // maximum2.hpp:41
  } else if (mode == kAbsMax || mode == kMaxMax) {
    const float hi = *M;
    *M = (hi > Mb) ? hi : Mb;
  } else if (mode == kMinMaxMva) {
    // MulScalar, MulScalar, Add2: three roundings per statistic
    const float a = decay * *m, b = one_minus_decay * mb;
    *m = a + b;
    const float c = decay * *M, d = one_minus_decay * Mb;
    *M = c + d;
  } else {
    const float c = decay * *M, d = one_minus_decay * Mb;
    *M = c + d;
  }
}

// Counters that tell a block whether it is the last of its launch to finish; one set per launch in flight (the host
// hands the slots out in turn).  Two levels, because a counter that every block of a grid updates is a serial chain
// of device-wide atomics (about 15 ns each): block b draws a ticket from counter b % kTicketGroups, and the block
// that draws the last ticket of a counter draws one from the set's final counter.  Zero when the module is loaded;
// the last block puts the zeros back.
// (Counters sit 256 bytes apart: atomics on one cache line queue up behind each other whatever their address.)
constexpr int kRecorderTickets = 16, kTicketGroups = 32, kTicketStride = 64;
__device__ unsigned g_recorder_tickets[kRecorderTickets][(kTicketGroups + 1) * kTicketStride];

// One launch scans (and copies) the array and updates the statistic.  Every block publishes its extrema with
// device-scope atomic stores, waits until the memory system has acknowledged them (vmcnt(0)) and draws a ticket;
// the block that draws the last one reads all the partial results back with atomic loads (they are complete: every
// other block's stores were acknowledged before its ticket), merges them in block order and applies the update.
// Only atomics carry the hand-over, so no cache is written back or invalidated.
// kAligned false: x (or y) does not start at a multiple of 16 bytes; a lane's four values then come and go as four
// 32-bit accesses.
template <bool kAbs, bool kCopy, bool kAligned>
__global__ __launch_bounds__(kRedBlock) void record_scan(const float *__restrict__ x, float *__restrict__ y,
                                                         MinMaxPartial *__restrict__ partial, size_t n4, size_t size,
                                                         float *__restrict__ m, float *__restrict__ M, int mode,
                                                         float decay, float one_minus_decay, int slot) {
  Extrema ex;
  ex.init();
  const size_t per = (n4 + gridDim.x - 1) / gridDim.x;
  const size_t begin = (size_t)blockIdx.x * per, end = (begin + per < n4) ? begin + per : n4;
  size_t i = begin + threadIdx.x;
  auto ld = [](const float *p) {
    return kAligned ? load4(p) : float4_t{p[0], p[1], p[2], p[3]};
  };
  auto st = [](float *p, float4_t v) {
    if (kAligned) {
      store4(p, v);
    } else {
      __builtin_nontemporal_store(v.x, p), __builtin_nontemporal_store(v.y, p + 1);
      __builtin_nontemporal_store(v.z, p + 2), __builtin_nontemporal_store(v.w, p + 3);
    }
  };
  auto absolute = [](float4_t v) {
    return float4_t{__builtin_fabsf(v.x), __builtin_fabsf(v.y), __builtin_fabsf(v.z), __builtin_fabsf(v.w)};
  };
  // four 16-byte loads per thread in flight while the previous four are consumed
  if (i + 3 * kRedBlock < end) {
    float4_t cur[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      cur[j] = ld(x + 4 * (i + j * kRedBlock));
#pragma clang loop unroll(disable)
    for (;;) {
      const size_t nx = i + 4 * kRedBlock;
      const bool more = nx + 3 * kRedBlock < end;
      float4_t nxt[4];
      if (more) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          nxt[j] = ld(x + 4 * (nx + j * kRedBlock));
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (kCopy)
          st(y + 4 * (i + j * kRedBlock), cur[j]);
        ex.take4(kAbs ? absolute(cur[j]) : cur[j], (uint32_t)(4 * (i + j * kRedBlock)));
      }
      i = nx;
      if (!more)
        break;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        cur[j] = nxt[j];
    }
  }
  for (; i < end; i += kRedBlock) {
    float4_t v = ld(x + 4 * i);
    if (kCopy)
      st(y + 4 * i, v);
    ex.take4(kAbs ? absolute(v) : v, (uint32_t)(4 * i));
  }
  if (blockIdx.x == gridDim.x - 1) { // the elements past the last float4 (all of them when n4 is 0), highest indices
    for (size_t t = 4 * n4 + threadIdx.x; t < size; t += kRedBlock) {
      const float v = x[t];
      if (kCopy)
        y[t] = v;
      ex.take(kAbs ? __builtin_fabsf(v) : v, (uint32_t)t);
    }
  }
  ex.wave_reduce();
  __shared__ MinMaxPartial s_part[kRedBlock / 64];
  __shared__ unsigned s_ticket;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0)
    s_part[wave] = ex.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRedBlock / 64; ++w)
      ex.merge(s_part[w].vmin, s_part[w].vmax, s_part[w].zidx, s_part[w].zsign);
    unsigned long long *dst = reinterpret_cast<unsigned long long *>(&partial[blockIdx.x]);
    const unsigned long long lo = (unsigned long long)__float_as_uint(ex.vmin) |
                                  ((unsigned long long)__float_as_uint(ex.vmax) << 32);
    const unsigned long long hi = (unsigned long long)ex.zidx | ((unsigned long long)ex.zsign << 32);
    __hip_atomic_store(dst, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(dst + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the two stores have been performed
    asm volatile("" ::: "memory");
    // 1 = this block is the last of the launch
    unsigned *tickets = g_recorder_tickets[slot];
    const unsigned groups = gridDim.x < (unsigned)kTicketGroups ? gridDim.x : (unsigned)kTicketGroups;
    const unsigned group = blockIdx.x % groups, members = (gridDim.x - group + groups - 1) / groups;
    unsigned last = 0u;
    if (atomicAdd(&tickets[group * kTicketStride], 1u) == members - 1u)
      last = atomicAdd(&tickets[kTicketGroups * kTicketStride], 1u) == groups - 1u ? 1u : 0u;
    s_ticket = last;
  }
  __syncthreads();
  if (s_ticket == 0u)
    return;
  // the last block: every thread takes the partial results c = thread, thread + 256, ... four at a time (eight loads
  // in flight: one round trip for up to 1024 blocks); the merge does not depend on the order
  Extrema all;
  all.init();
  for (unsigned c0 = threadIdx.x; c0 < gridDim.x; c0 += 4 * kRedBlock) {
    unsigned long long lo[4], hi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned c = c0 + j * kRedBlock;
      const unsigned long long *src = reinterpret_cast<const unsigned long long *>(&partial[c < gridDim.x ? c : c0]);
      lo[j] = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      hi[j] = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      all.merge(__uint_as_float((uint32_t)lo[j]), __uint_as_float((uint32_t)(lo[j] >> 32)), (uint32_t)hi[j],
                (uint32_t)(hi[j] >> 32));
  }
  all.wave_reduce();
  if (lane == 0)
    s_part[wave] = all.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRedBlock / 64; ++w)
      all.merge(s_part[w].vmin, s_part[w].vmax, s_part[w].zidx, s_part[w].zsign);
    record_apply(all, m, M, mode, decay, one_minus_decay);
  }
  if (threadIdx.x <= kTicketGroups)
    __hip_atomic_store(&g_recorder_tickets[slot][threadIdx.x * kTicketStride], 0u, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

} // namespace
} // namespace nbla_hip

extern "C" {

size_t nbla_hip_range_recorder_workspace_bytes(void) { return (size_t)kMaxChunks * sizeof(MinMaxPartial); }

int nbla_hip_range_recorder_f32(const float *x, float *y, size_t size, float *m, float *M, int mode, double decay,
                                int training, void *workspace, size_t workspace_bytes, void *stream_) {
  if (mode < 0 || mode >= kRecorderModes)
    return fail(NBLA_HIP_ERR_VALUE, "range recorder: unknown mode %d.", mode);
  if (size > 0xffffffffull)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "range recorder: arrays above 2^32 elements are not supported.");
  hipStream_t stream = as_stream(stream_);
  if (!training) { // y.copy_from(x) only
    if (size && y != x) {
      hipError_t e = hipMemcpyAsync(y, x, size * sizeof(float), hipMemcpyDeviceToDevice, stream);
      if (e != hipSuccess)
        return fail_hip(e, "range recorder copy");
    }
    return NBLA_HIP_OK;
  }
  const bool two = (mode == kMinMaxMinMax || mode == kMinMaxMva);
  if (M == nullptr || (two && m == nullptr))
    return fail(NBLA_HIP_ERR_VALUE, "range recorder: the statistics arrays are missing.");
  if (workspace_bytes < nbla_hip_range_recorder_workspace_bytes() || !aligned16(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "range recorder workspace too small or misaligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  MinMaxPartial *partial = static_cast<MinMaxPartial *>(workspace);
  const bool copy = (y != x);
  const bool aligned = aligned16(x) && (!copy || aligned16(y));
  const size_t n4 = size / 4;
  size_t blocks = (n4 + kRedBlock * 4 - 1) / (kRedBlock * 4);
  if (blocks > (size_t)kMaxChunks)
    blocks = kMaxChunks;
  if (blocks < 1)
    blocks = 1;
  const dim3 grid((unsigned)blocks), block(kRedBlock);
  // `decay * m` and `(1 - decay) * mb` of the reference are MulScalar functions: each takes the Python float (a
  // double) and rounds it to fp32 once
  const float dec = (float)decay, omd = (float)(1.0 - decay);
  static std::atomic<unsigned> next_slot{0};
  const int slot = (int)(next_slot.fetch_add(1u) % (unsigned)kRecorderTickets);
#define NBLA_RECORD_SCAN(ABS, COPY)                                                                                    \
  do {                                                                                                                 \
    if (aligned)                                                                                                       \
      hipLaunchKernelGGL((record_scan<ABS, COPY, true>), grid, block, 0, stream, x, y, partial, n4, size, m, M, mode,  \
                         dec, omd, slot);                                                                              \
    else                                                                                                               \
      hipLaunchKernelGGL((record_scan<ABS, COPY, false>), grid, block, 0, stream, x, y, partial, n4, size, m, M, mode, \
                         dec, omd, slot);                                                                              \
  } while (0)
  if (mode == kAbsMax) {
    if (copy)
      NBLA_RECORD_SCAN(true, true);
    else
      NBLA_RECORD_SCAN(true, false);
  } else {
    if (copy)
      NBLA_RECORD_SCAN(false, true);
    else
      NBLA_RECORD_SCAN(false, false);
  }
#undef NBLA_RECORD_SCAN
  NBLA_HIP_LAUNCH_CHECK("range recorder scan");
  return NBLA_HIP_OK;
}

} // extern "C"
