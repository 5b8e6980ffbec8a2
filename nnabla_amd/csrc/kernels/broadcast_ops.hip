// Two-input arithmetic with broadcasting (Add2 / Sub2 / Mul2 / Div2 / Pow2 on inputs of different shapes): what the
// reference computes through strides that are zero along a broadcast axis,
// include/nbla/function/utils/base_transform_binary.hpp:58-205 (shapes and strides), :265-284 (forward), :286-336
// (gradients, accumulated into the smaller operand).
//
// Adjacent axes that broadcast in the same way are merged (base_transform_binary.hpp:98-150), which leaves at most
// eight groups for eight axes.  Forward: one thread per output element, the two operand indices by division over the
// groups (32-bit when the element count allows).  Gradient of an operand that is not broadcast: the same, element by
// element.  Gradient of a broadcast operand: one block per element of the operand sums that element's terms -- they
// lie at the output positions the broadcast groups span, walked in ascending output index -- as 256 interleaved
// partial sums folded through LDS in a fixed order.  The reference adds the same terms one after the other in fp32
// (g[idx0] += ...), so the two sums agree to rounding, not to the bit; the result does not change from run to run.
#include "common.hpp"
#include "internal.hpp"

#include <math.h>

namespace nbla_hip {
namespace {

constexpr int kBlk = 256;
constexpr int kMaxGroups = 8;

struct Groups {
  int nd;
  int64_t shape[kMaxGroups];      // of the output
  int64_t sy[kMaxGroups];         // strides of the output
  int64_t s[2][kMaxGroups];       // strides of the operands, 0 along a broadcast group
  int64_t total, count[2];        // elements of the output, of the operands
};

enum { kSub = 0, kMul = 1, kDiv = 2, kAdd = 3, kPow = 4 };

// sub2.hpp:41, mul2.hpp:42, div2.hpp:44, add2.hpp (bc_add2.hpp), pow2.hpp:44-47
template <int kOp> __device__ __forceinline__ float forward_of(float x0, float x1) {
  switch (kOp) {
  case kSub: return x0 - x1;
  case kMul: return x0 * x1;
  case kDiv: return x0 / x1;
  case kAdd: return x0 + x1;
  default: return powf(x0, x1);
  }
}
template <int kOp, int kInput> __device__ __forceinline__ float grad_of(float dy, float x0, float x1) {
  switch (kOp) {
  case kSub: return kInput == 0 ? dy : -dy;
  case kMul: return kInput == 0 ? dy * x1 : dy * x0;
  case kDiv: return kInput == 0 ? dy / x1 : -dy * x0 / (x1 * x1);
  case kAdd: return dy;
  default: return kInput == 0 ? dy * x1 * powf(x0, x1 - 1.0f) : dy * logf(x0) * powf(x0, x1);
  }
}
template <int kOp> constexpr bool reads_inputs() { return kOp != kSub && kOp != kAdd; }

template <typename Index> __device__ __forceinline__ void operand_indices(const Groups &g, Index idx, int64_t &i0, int64_t &i1) {
  i0 = 0, i1 = 0;
#pragma unroll 1
  for (int d = g.nd - 1; d >= 0; --d) {
    const Index n = (Index)g.shape[d];
    const Index q = idx / n, r = idx - q * n;
    i0 += (int64_t)r * g.s[0][d];
    i1 += (int64_t)r * g.s[1][d];
    idx = q;
  }
}

template <int kOp, typename Index>
__global__ __launch_bounds__(kBlk) void broadcast2_forward(const float *__restrict__ x0, const float *__restrict__ x1,
                                                           float *__restrict__ y, Groups g) {
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < g.total; t += (int64_t)gridDim.x * kBlk) {
    int64_t i0, i1;
    operand_indices<Index>(g, (Index)t, i0, i1);
    y[t] = forward_of<kOp>(x0[i0], x1[i1]);
  }
}

// operand kInput has the output's shape
template <int kOp, int kInput, typename Index>
__global__ __launch_bounds__(kBlk) void broadcast2_grad_dense(const float *dy, const float *__restrict__ x0,
                                                              const float *__restrict__ x1, float *dx, Groups g,
                                                              int accum) {
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < g.total; t += (int64_t)gridDim.x * kBlk) {
    int64_t i0, i1;
    operand_indices<Index>(g, (Index)t, i0, i1);
    const float v = grad_of<kOp, kInput>(dy[t], reads_inputs<kOp>() ? x0[i0] : 0.0f, reads_inputs<kOp>() ? x1[i1] : 0.0f);
    dx[t] = (accum ? dx[t] : 0.0f) + v;
  }
}

// operand kInput is broadcast: block = one of its elements
template <int kOp, int kInput>
__global__ __launch_bounds__(kBlk) void broadcast2_grad_reduce(const float *__restrict__ dy, const float *__restrict__ x0,
                                                               const float *__restrict__ x1, float *__restrict__ dx,
                                                               Groups g, int accum) {
  __shared__ float part[kBlk];
  const int64_t j = blockIdx.x;
  // the element's own position: its index over the groups it is not broadcast along; the terms' positions: every
  // index over the groups it is broadcast along
  int64_t base_y = 0, base_other = 0, terms = 1;
  {
    int64_t rest = j;
    for (int d = g.nd - 1; d >= 0; --d) {
      if (g.s[kInput][d] == 0) {
        terms *= g.shape[d];
        continue;
      }
      const int64_t r = rest % g.shape[d];
      rest /= g.shape[d];
      base_y += r * g.sy[d];
      base_other += r * g.s[1 - kInput][d];
    }
  }
  float acc = 0.0f;
  for (int64_t t = threadIdx.x; t < terms; t += kBlk) {
    int64_t rest = t, iy = base_y, io = base_other;
    for (int d = g.nd - 1; d >= 0; --d) {
      if (g.s[kInput][d] != 0)
        continue;
      const int64_t r = rest % g.shape[d];
      rest /= g.shape[d];
      iy += r * g.sy[d];
      io += r * g.s[1 - kInput][d];
    }
    const float own = reads_inputs<kOp>() ? (kInput == 0 ? x0[j] : x1[j]) : 0.0f;
    const float other = reads_inputs<kOp>() ? (kInput == 0 ? x1[io] : x0[io]) : 0.0f;
    acc += grad_of<kOp, kInput>(dy[iy], kInput == 0 ? own : other, kInput == 0 ? other : own);
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int w = kBlk / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w)
      part[threadIdx.x] += part[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0)
    dx[j] = (accum ? dx[j] : 0.0f) + part[0];
}

// base_transform_binary.hpp:58-205: output shape, merged groups, strides
int make_groups(Groups &g, int ndim, const int64_t *shape0, const int64_t *shape1, const char *what) {
  if (ndim < 0 || ndim > 16)
    return fail(NBLA_HIP_ERR_VALUE, "%s: %d dimensions.", what, ndim);
  int64_t s0[16], s1[16], so[16];
  for (int i = 0; i < ndim; ++i) {
    s0[i] = shape0[i], s1[i] = shape1[i];
    if (s0[i] < 0 || s1[i] < 0)
      return fail(NBLA_HIP_ERR_VALUE, "%s: negative size at dimension %d.", what, i);
    if (s0[i] != s1[i] && (s0[i] < s1[i] ? s0[i] : s1[i]) != 1)
      return fail(NBLA_HIP_ERR_VALUE, "Broadcast dimension must be one. shape[%d]: %lld.", i,
                  (long long)(s0[i] < s1[i] ? s0[i] : s1[i]));
    so[i] = s0[i] > s1[i] ? s0[i] : s1[i];
  }
  int64_t c0[16], c1[16], cy[16];
  int n = 0;
  int64_t t0 = 1, t1 = 1, ty = 1;
  for (int i = 0; i + 1 < ndim; ++i) {
    t0 *= s0[i], t1 *= s1[i], ty *= so[i];
    auto kind = [&](int a) { return s0[a] == s1[a] ? 0 : (s0[a] == 1 ? 1 : 2); };
    if (kind(i) != kind(i + 1)) {
      c0[n] = t0, c1[n] = t1, cy[n] = ty;
      ++n;
      t0 = t1 = ty = 1;
    }
  }
  if (ndim > 0) {
    t0 *= s0[ndim - 1], t1 *= s1[ndim - 1], ty *= so[ndim - 1];
    c0[n] = t0, c1[n] = t1, cy[n] = ty;
    ++n;
  }
  if (n == 0) { // scalars
    c0[0] = c1[0] = cy[0] = 1;
    n = 1;
  }
  if (n > kMaxGroups)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "%s: more than %d groups of axes after merging.", what, kMaxGroups);
  g.nd = n;
  int64_t st0 = 1, st1 = 1, sty = 1;
  for (int d = n - 1; d >= 0; --d) {
    g.shape[d] = cy[d];
    g.sy[d] = sty;
    g.s[0][d] = c0[d] == cy[d] ? st0 : 0;
    g.s[1][d] = c1[d] == cy[d] ? st1 : 0;
    st0 *= c0[d], st1 *= c1[d], sty *= cy[d];
  }
  g.total = sty, g.count[0] = st0, g.count[1] = st1;
  return NBLA_HIP_OK;
}

unsigned blocks_for(int64_t n) {
  int64_t b = (n + kBlk - 1) / kBlk;
  return (unsigned)(b > 65536 ? 65536 : (b < 1 ? 1 : b));
}

template <int kOp> int forward(const float *x0, const float *x1, float *y, const Groups &g, hipStream_t s) {
  if (g.total < ((int64_t)1 << 31))
    hipLaunchKernelGGL((broadcast2_forward<kOp, uint32_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, x0, x1, y, g);
  else
    hipLaunchKernelGGL((broadcast2_forward<kOp, int64_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, x0, x1, y, g);
  NBLA_HIP_LAUNCH_CHECK("broadcast2 forward");
  return NBLA_HIP_OK;
}

template <int kOp, int kInput>
int backward(const float *dy, const float *x0, const float *x1, float *dx, const Groups &g, int accum, hipStream_t s) {
  if (g.count[kInput] == g.total) {
    if (g.total < ((int64_t)1 << 31))
      hipLaunchKernelGGL((broadcast2_grad_dense<kOp, kInput, uint32_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, dy,
                         x0, x1, dx, g, accum);
    else
      hipLaunchKernelGGL((broadcast2_grad_dense<kOp, kInput, int64_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, dy,
                         x0, x1, dx, g, accum);
  } else {
    if (g.count[kInput] > 0x7fffffffll)
      return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "broadcast2 backward: a broadcast operand of 2^31 elements or more.");
    hipLaunchKernelGGL((broadcast2_grad_reduce<kOp, kInput>), dim3((unsigned)g.count[kInput]), dim3(kBlk), 0, s, dy, x0,
                       x1, dx, g, accum);
  }
  NBLA_HIP_LAUNCH_CHECK("broadcast2 backward");
  return NBLA_HIP_OK;
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_broadcast2_f32(int op, const float *x0, const int64_t *shape0, const float *x1, const int64_t *shape1,
                            float *y, int ndim, void *stream) {
  Groups g;
  const int rc = make_groups(g, ndim, shape0, shape1, "broadcast2");
  if (rc)
    return rc;
  if (g.total == 0)
    return NBLA_HIP_OK;
  hipStream_t s = as_stream(stream);
  switch (op) {
  case kSub: return forward<kSub>(x0, x1, y, g, s);
  case kMul: return forward<kMul>(x0, x1, y, g, s);
  case kDiv: return forward<kDiv>(x0, x1, y, g, s);
  case kAdd: return forward<kAdd>(x0, x1, y, g, s);
  case kPow: return forward<kPow>(x0, x1, y, g, s);
  }
  return fail(NBLA_HIP_ERR_VALUE, "broadcast2: unknown operation %d.", op);
}

int nbla_hip_broadcast2_backward_f32(int op, int input, const float *dy, const float *x0, const int64_t *shape0,
                                     const float *x1, const int64_t *shape1, float *dx, int ndim, int accum,
                                     void *stream) {
  if (input != 0 && input != 1)
    return fail(NBLA_HIP_ERR_VALUE, "broadcast2 backward: input %d is not 0 or 1.", input);
  Groups g;
  const int rc = make_groups(g, ndim, shape0, shape1, "broadcast2 backward");
  if (rc)
    return rc;
  if (g.count[input] == 0 || (g.total == 0 && g.count[input] == g.total))
    return NBLA_HIP_OK;
  hipStream_t s = as_stream(stream);
#define NBLA_BROADCAST2_GRAD(OP)                                                                                       \
  return input == 0 ? backward<OP, 0>(dy, x0, x1, dx, g, accum, s) : backward<OP, 1>(dy, x0, x1, dx, g, accum, s)
  switch (op) {
  case kSub: NBLA_BROADCAST2_GRAD(kSub);
  case kMul: NBLA_BROADCAST2_GRAD(kMul);
  case kDiv: NBLA_BROADCAST2_GRAD(kDiv);
  case kAdd: NBLA_BROADCAST2_GRAD(kAdd);
  case kPow: NBLA_BROADCAST2_GRAD(kPow);
  }
#undef NBLA_BROADCAST2_GRAD
  return fail(NBLA_HIP_ERR_VALUE, "broadcast2 backward: unknown operation %d.", op);
}

} // extern "C"
