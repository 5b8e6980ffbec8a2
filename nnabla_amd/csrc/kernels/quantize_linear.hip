// QuantizeLinear, DequantizeLinear (broadcast scale / zero point, each arithmetic step rounded on its own as the
// reference's chain of Div2 / round / Add2 / saturate does) and Prune (k-th smallest |x| by a three-pass radix
// select over the magnitude bits, then a masked copy).  All HBM-bound; 128-bit accesses where the layout allows.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "quantize_common.hpp"
#include "radix_select.hpp"

#include <cmath>

namespace nbla_hip {
namespace {

typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

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

template <typename Index>
__device__ __forceinline__ void offsets(const Broadcast &b, Index i, int64_t &so, int64_t &zo) {
  so = zo = 0;
#pragma unroll
  for (int d = kMaxDims - 1; d >= 0; --d) {
    if (d < b.nd) {
      const Index q = (d == 0) ? 0 : i / (Index)b.size[d];
      const Index c = (d == 0) ? i : i - q * (Index)b.size[d];
      so += (int64_t)c * b.sstride[d];
      zo += (int64_t)c * b.zstride[d];
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

// x / s.  A scale that is a power of two with a normal reciprocal is divided by multiplying with that reciprocal:
// both are the one correct rounding of the same real number.
__device__ __forceinline__ float divide(float x, float s) {
  const uint32_t u = __float_as_uint(s), e = u >> 23;
  if ((u & 0x807fffffu) == 0u && e >= 1u && e <= 253u)
    return x * __uint_as_float((254u - e) << 23);
  return x / s;
}

// round(x / s) as far as saturate(. + zero_point) to an 8-bit range can tell.  The quotient is first estimated with
// the hardware reciprocal (within 3 ulp of the true quotient, so within 3.5 ulp of its fp32 rounding).  Unless the
// estimate lies within 8 ulp of a rounding tie k + 1/2, it and the correctly rounded quotient round to the same
// integer; estimates of magnitude >= 4096 saturate whatever their last bits are (|zero_point| <= 255).  Everything
// else (near-ties, NaN, scales whose reciprocal is not a normal number) takes the IEEE division.
__device__ __forceinline__ float rounded_quotient(float x, float s, int half_to_even) {
  const float a = fabsf(s);
  if (a >= 0x1p-100f && a <= 0x1p100f) {
    const float q = x * __builtin_amdgcn_rcpf(s);
    const float t = rintf(q); // away from a tie every rounding mode gives this integer (and the same signed zero)
    const float m = fabsf(q);
    const float d = 0.5f - fabsf(q - t); // distance from the nearest tie; q - t is exact below 2^23
    if (m >= 4096.0f || d > fmaxf(m, 0.5f) * 0x1p-20f)
      return t;
  }
  return round_mode(divide(x, s), half_to_even);
}

struct QuantizeOp {
  static constexpr bool kRoundsZeroPoint = false;
  static constexpr bool kUniform = false;
  int half_to_even;
  float lo, hi;
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const {
    return saturate(rounded_quotient(x, scale, half_to_even) + zp, lo, hi);
  }
};
// The same with a one-element zero point that has not been rounded yet: every thread rounds it for itself and one
// thread stores the rounded value back (quantize_linear.cpp:109-111 rounds the zero point in place).  Threads that
// read it after that store find a value rounding leaves unchanged.
struct QuantizeRoundingOp {
  static constexpr bool kRoundsZeroPoint = true;
  static constexpr bool kUniform = false;
  int half_to_even;
  float lo, hi;
  __device__ __forceinline__ float zero_point(float zp) const { return saturate(round_mode(zp, half_to_even), lo, hi); }
  // zp: already rounded by the caller (once per thread)
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const {
    return saturate(rounded_quotient(x, scale, half_to_even) + zp, lo, hi);
  }
};
// One scale and one zero point for the whole tensor (what per-tensor quantization-aware training produces): the
// reciprocal, the range check of the scale and the rounded zero point are worked out once per thread, and no
// broadcast offsets are computed.
struct QuantizeUniformOp {
  static constexpr bool kRoundsZeroPoint = false;
  static constexpr bool kUniform = true;
  int half_to_even;
  float lo, hi;
  struct State {
    float s, inv, zp;
    bool fast;
  };
  __device__ __forceinline__ State prepare(float s, float zp_raw) const {
    State st;
    const float a = fabsf(s);
    st.s = s;
    st.fast = a >= 0x1p-100f && a <= 0x1p100f;
    st.inv = st.fast ? __builtin_amdgcn_rcpf(s) : 0.0f;
    st.zp = saturate(round_mode(zp_raw, half_to_even), lo, hi);
    return st;
  }
  __device__ __forceinline__ float apply(float x, const State &st) const { // rounded_quotient with the shared parts
    if (st.fast) {
      const float q = x * st.inv;
      const float t = rintf(q);
      const float m = fabsf(q);
      const float d = 0.5f - fabsf(q - t);
      if (m >= 4096.0f || d > fmaxf(m, 0.5f) * 0x1p-20f)
        return saturate(t + st.zp, lo, hi);
    }
    return saturate(round_mode(divide(x, st.s), half_to_even) + st.zp, lo, hi);
  }
  // Four values at once: the estimate's rounding for all of them, then one (rare, divergent) branch for those near a
  // tie instead of one per value -- the execution-mask bookkeeping of sixteen branches per thread cost more than the
  // arithmetic.
  __device__ __forceinline__ float4_t apply4(float4_t x, const State &st) const {
    float4_t r;
    if (st.fast) { // uniform
      bool near[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float q = x[e] * st.inv;
        const float t = rintf(q);
        const float m = fabsf(q);
        const float d = 0.5f - fabsf(q - t);
        near[e] = !(m >= 4096.0f || d > fmaxf(m, 0.5f) * 0x1p-20f);
        r[e] = saturate(t + st.zp, lo, hi);
      }
      if (near[0] | near[1] | near[2] | near[3]) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (near[e])
            r[e] = saturate(round_mode(divide(x[e], st.s), half_to_even) + st.zp, lo, hi);
      }
      return r;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      r[e] = saturate(round_mode(divide(x[e], st.s), half_to_even) + st.zp, lo, hi);
    return r;
  }
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const { return 0.0f; } // not used
};
struct DequantizeOp {
  static constexpr bool kRoundsZeroPoint = false;
  static constexpr bool kUniform = false;
  __device__ __forceinline__ float operator()(float x, float scale, float zp) const { return (x - zp) * scale; }
};
// dx (+)= dy / scale  and  dx (+)= dy * scale  (the zero point is not read)
struct DivGradOp {
  static constexpr bool kRoundsZeroPoint = false;
  static constexpr bool kUniform = false;
  __device__ __forceinline__ float operator()(float dy, float scale, float) const { return divide(dy, scale); }
};
struct MulGradOp {
  static constexpr bool kRoundsZeroPoint = false;
  static constexpr bool kUniform = false;
  __device__ __forceinline__ float operator()(float dy, float scale, float) const { return dy * scale; }
};

// y[i] = op(x[i], scale[...], zp[...]) (+ y[i] when kAccum).  kVec: four float4 per thread (loads issued together),
// each float4 inside the innermost dimension (its size is a multiple of four).  Index: uint32_t when the element
// count fits, so the index decomposition divides in 32 bits.
constexpr int kUnroll = 4;
template <typename Op, bool kVec, bool kAccum, typename Index>
__global__ __launch_bounds__(kBlock) void broadcast_map(const float *__restrict__ x, const float *__restrict__ scale,
                                                        const float *__restrict__ zp, float *__restrict__ y,
                                                        int64_t count, Broadcast b, Op op) {
  if constexpr (Op::kUniform) {
    const auto st = op.prepare(scale[0], zp[0]);
    if (blockIdx.x == 0 && threadIdx.x == 0)
      const_cast<float *>(zp)[0] = st.zp;
    if (kVec) {
      const int64_t base = (int64_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
      float4_t v[kUnroll];
#pragma unroll
      for (int j = 0; j < kUnroll; ++j)
        if (base + (int64_t)j * kBlock < count)
          v[j] = *reinterpret_cast<const float4_t *>(x + 4 * (base + (int64_t)j * kBlock));
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        const int64_t t = base + (int64_t)j * kBlock;
        if (t < count) {
          const float4_t o = op.apply4(v[j], st);
          __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(y + 4 * t));
        }
      }
    } else {
      const int64_t step = (int64_t)gridDim.x * kBlock;
      for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < count; t += step)
        y[t] = op.apply(x[t], st);
    }
    return;
  }
  float rounded_zp = 0.0f;
  if constexpr (Op::kRoundsZeroPoint) {
    rounded_zp = op.zero_point(zp[0]);
    if (blockIdx.x == 0 && threadIdx.x == 0)
      const_cast<float *>(zp)[0] = rounded_zp;
  }
  if (kVec) {
    const int64_t base = (int64_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
    float4_t v[kUnroll], old[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      const int64_t t = base + (int64_t)j * kBlock;
      if (t < count) {
        v[j] = *reinterpret_cast<const float4_t *>(x + 4 * t);
        if (kAccum)
          old[j] = *reinterpret_cast<const float4_t *>(y + 4 * t);
      }
    }
    const int64_t ss = b.sstride[b.nd - 1], zs = b.zstride[b.nd - 1];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      const int64_t t = base + (int64_t)j * kBlock;
      if (t < count) {
        int64_t so, zo;
        offsets<Index>(b, (Index)(4 * t), so, zo);
        // innermost stride 0: one value for the four elements; stride 1: four consecutive values
        float4_t sv, zv;
        if (ss == 0)
          sv.x = sv.y = sv.z = sv.w = scale[so];
        else
          sv = *reinterpret_cast<const float4_t *>(scale + so);
        if (Op::kRoundsZeroPoint)
          zv.x = zv.y = zv.z = zv.w = rounded_zp;
        else if (!zp)
          zv.x = zv.y = zv.z = zv.w = 0.0f;
        else if (zs == 0)
          zv.x = zv.y = zv.z = zv.w = zp[zo];
        else
          zv = *reinterpret_cast<const float4_t *>(zp + zo);
        float4_t o;
        o.x = op(v[j].x, sv.x, zv.x);
        o.y = op(v[j].y, sv.y, zv.y);
        o.z = op(v[j].z, sv.z, zv.z);
        o.w = op(v[j].w, sv.w, zv.w);
        if (kAccum)
          o.x = old[j].x + o.x, o.y = old[j].y + o.y, o.z = old[j].z + o.z, o.w = old[j].w + o.w;
        __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(y + 4 * t));
      }
    }
  } else {
    const int64_t step = (int64_t)gridDim.x * kBlock;
    for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < count; t += step) {
      int64_t so, zo;
      offsets<Index>(b, (Index)t, so, zo);
      const float o = op(x[t], scale[so], Op::kRoundsZeroPoint ? rounded_zp : (zp ? zp[zo] : 0.0f));
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
  const bool vec = b.size[b.nd - 1] % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(scale) && aligned16(zp);
  const bool narrow = total < ((int64_t)1 << 31);
  const int64_t count = vec ? total / 4 : total;
  int64_t blocks = ceil_div(count, (int64_t)kBlock * (vec ? kUnroll : 1));
  if (!vec && blocks > 1048576)
    blocks = 1048576; // grid-stride loop
#define NBLA_LAUNCH_MAP(V, A, I)                                                                                       \
  hipLaunchKernelGGL((broadcast_map<Op, V, A, I>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, x, scale, zp, y,   \
                     count, b, op)
#define NBLA_LAUNCH_MAP_I(V, A)                                                                                        \
  do {                                                                                                                 \
    if (narrow)                                                                                                        \
      NBLA_LAUNCH_MAP(V, A, uint32_t);                                                                                 \
    else                                                                                                               \
      NBLA_LAUNCH_MAP(V, A, int64_t);                                                                                  \
  } while (0)
  if (vec && accum)
    NBLA_LAUNCH_MAP_I(true, true);
  else if (vec)
    NBLA_LAUNCH_MAP_I(true, false);
  else if (accum)
    NBLA_LAUNCH_MAP_I(false, true);
  else
    NBLA_LAUNCH_MAP_I(false, false);
#undef NBLA_LAUNCH_MAP_I
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

// The rank-th smallest magnitude by the radix select of radix_select.hpp: keys are the 31 magnitude bits of x.  The
// launches form a chain (three histogram passes, then the pass that writes y); each resolves the histogram its
// predecessor left behind, every block for itself, while its first loads are already under way.
//
// The second pass also keeps the keys it counts -- those that share the first digit with the rank-th smallest, a few
// percent of the data at most unless the magnitudes crowd into one binade -- in a per-block region of the workspace,
// and the third pass reads those instead of x.  A block whose region is too small for its share (values of one
// magnitude range clustered in one stretch of x) raises a flag, and the third pass then reads x as the others do.
constexpr int kPruneLoads = 4;          // 16-byte loads per thread in flight
constexpr int kCandPerBlock = 8192;     // candidate keys a block can keep
struct PruneState {
  SelectState sel;
  uint32_t overflow;                    // some block found more candidates than its region holds
  uint32_t counts[kSelectBlocks];       // candidates kept by each block of the second pass
  uint32_t pad[3];
  uint32_t cand[kSelectBlocks][kCandPerBlock];
};

// kAligned false: x (or y) does not start at a multiple of 16 bytes; four 32-bit accesses per lane instead of one
// 128-bit access.
template <bool kAligned>
__device__ __forceinline__ void prune_fetch(const float *__restrict__ x, int64_t n4, int64_t tile,
                                            float4_t (&v)[kPruneLoads]) {
  const int64_t base = tile * (kHistBlock * kPruneLoads) + threadIdx.x;
#pragma unroll
  for (int j = 0; j < kPruneLoads; ++j)
    if (base + j * kHistBlock < n4) {
      const float *src = x + 4 * (base + j * kHistBlock);
      if (kAligned)
        v[j] = *reinterpret_cast<const float4_t *>(src);
      else
        v[j] = float4_t{src[0], src[1], src[2], src[3]};
    }
}

template <bool kAligned>
__global__ __launch_bounds__(kHistBlock) void prune_histogram(const float *__restrict__ x, int64_t n4, int64_t n,
                                                          PruneState *__restrict__ ps, int pass) {
  __shared__ uint32_t h[kMaxBins * kLdsCopies];
  __shared__ uint32_t scratch[kSelectScratch];
  __shared__ uint32_t s_kept;
  SelectState *st = &ps->sel;
  const int64_t tiles = (n4 + kHistBlock * kPruneLoads - 1) / (kHistBlock * kPruneLoads);
  const bool from_cand = pass == 2 && ps->overflow == 0u; // uniform over the grid
  const bool any = (int64_t)blockIdx.x < tiles && !from_cand;
  float4_t cur[kPruneLoads];
  if (any)
    prune_fetch<kAligned>(x, n4, blockIdx.x, cur);
  if (threadIdx.x == 0) {
    s_kept = 0u;
    if (pass == 0 && blockIdx.x == 0)
      ps->overflow = 0u;
  }
  const SelectPass sp = select_begin_at(h, select_resolve(scratch, st, pass), pass);
  uint32_t *mine = ps->cand[blockIdx.x];
  auto count = [&](float v) {
    const uint32_t key = __float_as_uint(v) & 0x7fffffffu;
    if (pass == 1) { // (only the few elements behind the last whole 16 bytes come this way in the second pass)
      if ((key >> sp.above) == sp.want) {
        atomicAdd(&h[((key >> sp.shift) & sp.mask) * kLdsCopies + sp.copy], 1u);
        const uint32_t i = atomicAdd(&s_kept, 1u);
        if (i < (uint32_t)kCandPerBlock)
          mine[i] = key;
      }
    } else {
      select_count(h, sp, key);
    }
  };
  // Second pass, one tile: count the keys that share the first digit and keep them.  Nearly all keys do not, so
  // they are found without branches; a wavefront reserves room in the block's region for all its keys of the tile
  // with one LDS atomic (a counter bumped once per key is a serial chain).
  auto count_and_keep = [&](const float4_t (&v)[kPruneLoads], int64_t base) __attribute__((always_inline)) {
    uint32_t found = 0u; // bit 4 j + e: element e of load j shares the digit
#pragma unroll
    for (int j = 0; j < kPruneLoads; ++j) {
      const float e4[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
      const bool live = base + j * kHistBlock < n4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t key = __float_as_uint(e4[e]) & 0x7fffffffu;
        found |= (live && (key >> sp.above) == sp.want) ? 1u << (4 * j + e) : 0u;
      }
    }
    if (__ballot(found != 0u) == 0ull)
      return;
    const int lane = threadIdx.x & 63;
    const uint32_t c = (uint32_t)__popc(found);
    uint32_t incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off)
        incl += up;
    }
    uint32_t start = 0u;
    if (lane == 63)
      start = atomicAdd(&s_kept, incl);
    uint32_t at = (uint32_t)__shfl((int)start, 63) + incl - c;
#pragma unroll
    for (int j = 0; j < kPruneLoads; ++j) {
      const float e4[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (found & (1u << (4 * j + e))) {
          const uint32_t key = __float_as_uint(e4[e]) & 0x7fffffffu;
          atomicAdd(&h[((key >> sp.shift) & sp.mask) * kLdsCopies + sp.copy], 1u);
          if (at < (uint32_t)kCandPerBlock)
            mine[at] = key;
          ++at;
        }
    }
  };
  if (from_cand) {
    const uint32_t kept = ps->counts[blockIdx.x];
    for (uint32_t i = threadIdx.x; i < kept; i += kHistBlock)
      select_count(h, sp, mine[i]);
  }
  if (any) {
#pragma clang loop unroll(disable)
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
      const int64_t next = tile + gridDim.x;
      float4_t nxt[kPruneLoads];
      if (next < tiles)
        prune_fetch<kAligned>(x, n4, next, nxt);
      const int64_t base = tile * (kHistBlock * kPruneLoads) + threadIdx.x;
      if (pass == 1) {
        count_and_keep(cur, base);
      } else {
#pragma unroll
        for (int j = 0; j < kPruneLoads; ++j)
          if (base + j * kHistBlock < n4)
            count(cur[j].x), count(cur[j].y), count(cur[j].z), count(cur[j].w);
      }
#pragma unroll
      for (int j = 0; j < kPruneLoads; ++j)
        cur[j] = nxt[j];
    }
  }
  if (blockIdx.x == 0 && !from_cand) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < n)
      count(x[i]);
  }
  select_flush(h, st, sp); // (starts with a barrier: s_kept is final after it)
  if (pass == 1 && threadIdx.x == 0) {
    const uint32_t kept = s_kept;
    ps->counts[blockIdx.x] = kept < (uint32_t)kCandPerBlock ? kept : (uint32_t)kCandPerBlock;
    if (kept > (uint32_t)kCandPerBlock)
      ps->overflow = 1u;
  }
}

// y = (|x| < thresh) ? 0 : x with thresh = |rank-th smallest| (+ 1 when rate == 1), prune.cpp:62-69
template <bool kAligned>
__global__ __launch_bounds__(kHistBlock) void prune_apply(const float *__restrict__ x, float *__restrict__ y,
                                                          int64_t n4, int64_t n, PruneState *__restrict__ ps,
                                                          float add) {
  __shared__ uint32_t scratch[kSelectScratch];
  SelectState *st = &ps->sel;
  const int64_t tiles = (n4 + kHistBlock * kPruneLoads - 1) / (kHistBlock * kPruneLoads);
  const bool any = (int64_t)blockIdx.x < tiles;
  float4_t cur[kPruneLoads];
  if (any)
    prune_fetch<kAligned>(x, n4, blockIdx.x, cur);
  const float thresh = __uint_as_float(select_resolve(scratch, st, kPasses).prefix) + add;
  if (any) {
#pragma clang loop unroll(disable)
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
      const int64_t next = tile + gridDim.x;
      float4_t nxt[kPruneLoads];
      if (next < tiles)
        prune_fetch<kAligned>(x, n4, next, nxt);
      const int64_t base = tile * (kHistBlock * kPruneLoads) + threadIdx.x;
#pragma unroll
      for (int j = 0; j < kPruneLoads; ++j)
        if (base + j * kHistBlock < n4) {
          float4_t o;
          o.x = fabsf(cur[j].x) < thresh ? 0.0f : cur[j].x;
          o.y = fabsf(cur[j].y) < thresh ? 0.0f : cur[j].y;
          o.z = fabsf(cur[j].z) < thresh ? 0.0f : cur[j].z;
          o.w = fabsf(cur[j].w) < thresh ? 0.0f : cur[j].w;
          float *dst = y + 4 * (base + j * kHistBlock);
          if (kAligned) {
            __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(dst));
          } else {
            __builtin_nontemporal_store(o.x, dst), __builtin_nontemporal_store(o.y, dst + 1);
            __builtin_nontemporal_store(o.z, dst + 2), __builtin_nontemporal_store(o.w, dst + 3);
          }
        }
#pragma unroll
      for (int j = 0; j < kPruneLoads; ++j)
        cur[j] = nxt[j];
    }
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
  int64_t xsize = 1;
  for (int i = 0; i < ndim; ++i)
    xsize *= xshape[i];
  int64_t ssize = 1;
  for (int i = 0; i < ndim; ++i)
    ssize *= scale_shape[i];
  if (zsize == 1 && ssize == 1 && xsize > 0) {
    QuantizeUniformOp op{half_to_even ? 1 : 0, lo, hi};
    return launch_broadcast(x, scale, zero_point, y, xshape, scale_shape, zero_point_shape, ndim, false, op, stream,
                            "QuantizeLinear");
  }
  if (zsize == 1 && xsize > 0) { // no separate launch for the zero point
    QuantizeRoundingOp op{half_to_even ? 1 : 0, lo, hi};
    return launch_broadcast(x, scale, zero_point, y, xshape, scale_shape, zero_point_shape, ndim, false, op, stream,
                            "QuantizeLinear");
  }
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

size_t nbla_hip_prune_workspace_bytes(void) { return round_up(sizeof(PruneState), 256); }

int nbla_hip_prune_f32(const float *x, float *y, size_t size, float rate, void *workspace, size_t workspace_bytes,
                       void *stream_) {
  if (!(rate >= 0.0f && rate <= 1.0f))
    return fail(NBLA_HIP_ERR_VALUE, "Rate %f must be in [0, 1].", (double)rate);
  if (size == 0)
    return NBLA_HIP_OK;
  if (size > 0x7fffffffu)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "Prune: more than 2^31 - 1 elements (the reference indexes with int).");
  if (workspace_bytes < sizeof(PruneState) || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "Prune workspace too small or misaligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  PruneState *ps = static_cast<PruneState *>(workspace);
  SelectState *st = &ps->sel;
  // prune.cpp:33-34: thresh_idx_ = (int)((x_size - 1) * rate_), an int times a float
  const int x_size = (int)size;
  const uint32_t rank = (uint32_t)(int)((x_size - 1) * rate);
  const int64_t n = (int64_t)size;
  const int64_t n4 = n / 4;
  int64_t blocks = ceil_div(n4 ? n4 : 1, (int64_t)kHistBlock * kPruneLoads);
  if (blocks > kSelectBlocks)
    blocks = kSelectBlocks;
  hipLaunchKernelGGL(clear_select, dim3(clear_select_blocks()), dim3(256), 0, stream, st, rank);
  NBLA_HIP_LAUNCH_CHECK("clear_select");
  const bool aligned = aligned16(x) && aligned16(y);
  for (int p = 0; p < kPasses; ++p) {
    if (aligned)
      hipLaunchKernelGGL(prune_histogram<true>, dim3((unsigned)blocks), dim3(kHistBlock), 0, stream, x, n4, n, ps, p);
    else
      hipLaunchKernelGGL(prune_histogram<false>, dim3((unsigned)blocks), dim3(kHistBlock), 0, stream, x, n4, n, ps, p);
    NBLA_HIP_LAUNCH_CHECK("prune_histogram");
  }
  // every block of this launch resolves the last histogram first: two blocks per CU at most
  int64_t ablocks = ceil_div(n4 ? n4 : 1, (int64_t)kHistBlock * kPruneLoads);
  if (ablocks > 2 * kSelectBlocks)
    ablocks = 2 * kSelectBlocks;
  if (aligned)
    hipLaunchKernelGGL(prune_apply<true>, dim3((unsigned)ablocks), dim3(kHistBlock), 0, stream, x, y, n4, n, ps,
                       rate == 1.0f ? 1.0f : 0.0f);
  else
    hipLaunchKernelGGL(prune_apply<false>, dim3((unsigned)ablocks), dim3(kHistBlock), 0, stream, x, y, n4, n, ps,
                       rate == 1.0f ? 1.0f : 0.0f);
  NBLA_HIP_LAUNCH_CHECK("prune_apply");
  return NBLA_HIP_OK;
}

} // extern "C"
