// Two-input arithmetic with broadcasting (Add2 / Sub2 / Mul2 / Div2 / Pow2 on inputs of different shapes): what the
// reference computes through strides that are zero along a broadcast axis,
// include/nbla/function/utils/base_transform_binary.hpp:58-205 (shapes and strides), :265-284 (forward), :286-336
// (gradients, accumulated into the smaller operand).
//
// Adjacent axes that broadcast in the same way are merged (base_transform_binary.hpp:98-150), which leaves at most
// eight groups for eight axes.  Forward: one thread per output element, the two operand indices by division over the
// groups (32-bit, by multiplication with a precomputed reciprocal, when the element count allows; four consecutive
// elements per thread where the innermost group is a multiple of four and the pointers are aligned).  Gradient of an
// operand that is not broadcast: the same, element by element.  Gradient of a broadcast operand: a strided sum of the
// terms over the groups the operand is broadcast along, in one of two forms -- lanes along the operand's innermost
// kept group (a bias over the last axis), or lanes along the innermost run of terms (a bias per channel, a scalar) --
// with the terms of an element split over blocks where the elements are few, partial sums folded in a fixed order.
// Without a workspace: one block per element of the operand.  The reference adds the same terms one after the other
// in fp32 (g[idx0] += ...), so the sums agree to rounding, not to the bit; the result does not change from run to
// run.
#include "common.hpp"
#include "internal.hpp"
#include "quantize_common.hpp"

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
// 32-bit indices (fewer than 2^31 elements): the quotients by multiplication, n / d = (n * magic[d]) >> shift[d]
// exactly for n < 2^31 (magic = floor(2^shift / d) + 1, shift = 31 + ceil(log2 d)).
struct Reciprocals {
  uint32_t magic[kMaxGroups];
  int shift[kMaxGroups];
};
__device__ __forceinline__ void operand_indices_fast(const Groups &g, const Reciprocals &rc, uint32_t idx, int64_t &i0,
                                                     int64_t &i1) {
  i0 = 0, i1 = 0;
#pragma unroll 1
  for (int d = g.nd - 1; d >= 0; --d) {
    const uint32_t q = (uint32_t)(((uint64_t)idx * rc.magic[d]) >> rc.shift[d]);
    const uint32_t r = idx - q * (uint32_t)g.shape[d];
    i0 += (int64_t)r * g.s[0][d];
    i1 += (int64_t)r * g.s[1][d];
    idx = q;
  }
}

typedef float float4_v __attribute__((ext_vector_type(4)));

template <int kOp, typename Index>
__global__ __launch_bounds__(kBlk) void broadcast2_forward(const float *__restrict__ x0, const float *__restrict__ x1,
                                                           float *__restrict__ y, Groups g) {
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < g.total; t += (int64_t)gridDim.x * kBlk) {
    int64_t i0, i1;
    operand_indices<Index>(g, (Index)t, i0, i1);
    y[t] = forward_of<kOp>(x0[i0], x1[i1]);
  }
}
// Four consecutive elements of the innermost group per thread (its extent a multiple of four, fewer than 2^31
// elements, 16-byte aligned pointers): an operand is either contiguous along them or one value for all four.
template <int kOp>
__global__ __launch_bounds__(kBlk) void broadcast2_forward4(const float *__restrict__ x0, const float *__restrict__ x1,
                                                            float *__restrict__ y, Groups g, Reciprocals rc) {
  const int64_t n4 = g.total / 4;
  const bool run0 = g.s[0][g.nd - 1] != 0, run1 = g.s[1][g.nd - 1] != 0;
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < n4; t += (int64_t)gridDim.x * kBlk) {
    int64_t i0, i1;
    operand_indices_fast(g, rc, (uint32_t)(4 * t), i0, i1);
    float4_v a, b, r;
    if (run0)
      a = *reinterpret_cast<const float4_v *>(x0 + i0);
    else
      a = float4_v{x0[i0], x0[i0], x0[i0], x0[i0]};
    if (run1)
      b = *reinterpret_cast<const float4_v *>(x1 + i1);
    else
      b = float4_v{x1[i1], x1[i1], x1[i1], x1[i1]};
    r.x = forward_of<kOp>(a.x, b.x), r.y = forward_of<kOp>(a.y, b.y);
    r.z = forward_of<kOp>(a.z, b.z), r.w = forward_of<kOp>(a.w, b.w);
    __builtin_nontemporal_store(r, reinterpret_cast<float4_v *>(y + 4 * t));
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
template <int kOp, int kInput>
__global__ __launch_bounds__(kBlk) void broadcast2_grad_dense4(const float *dy, const float *__restrict__ x0,
                                                               const float *__restrict__ x1, float *dx, Groups g,
                                                               Reciprocals rc, int accum) {
  const int64_t n4 = g.total / 4;
  const bool run0 = g.s[0][g.nd - 1] != 0, run1 = g.s[1][g.nd - 1] != 0;
  const float4_v zero = float4_v{0.0f, 0.0f, 0.0f, 0.0f};
  for (int64_t t = (int64_t)blockIdx.x * kBlk + threadIdx.x; t < n4; t += (int64_t)gridDim.x * kBlk) {
    const float4_v gy = *reinterpret_cast<const float4_v *>(dy + 4 * t);
    float4_v a = zero, b = zero, r;
    if (reads_inputs<kOp>()) {
      int64_t i0, i1;
      operand_indices_fast(g, rc, (uint32_t)(4 * t), i0, i1);
      if (run0)
        a = *reinterpret_cast<const float4_v *>(x0 + i0);
      else
        a = float4_v{x0[i0], x0[i0], x0[i0], x0[i0]};
      if (run1)
        b = *reinterpret_cast<const float4_v *>(x1 + i1);
      else
        b = float4_v{x1[i1], x1[i1], x1[i1], x1[i1]};
    }
    const float4_v old = accum ? *reinterpret_cast<const float4_v *>(dx + 4 * t) : zero;
    r.x = old.x + grad_of<kOp, kInput>(gy.x, a.x, b.x), r.y = old.y + grad_of<kOp, kInput>(gy.y, a.y, b.y);
    r.z = old.z + grad_of<kOp, kInput>(gy.z, a.z, b.z), r.w = old.w + grad_of<kOp, kInput>(gy.w, a.w, b.w);
    *reinterpret_cast<float4_v *>(dx + 4 * t) = r;
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

// ---- the gradient of a broadcast operand as a strided sum.  The output (dy) seen from operand kInput: kept axes
// (the groups the operand spans; the operand's own index is row-major over them) and reduced axes (the groups it is
// broadcast along: the terms of one element), with the other operand's strides along both.
struct SumAxes {
  MinMaxAxes A;               // sizes and strides in dy
  int64_t ok[8], orr[8];      // the other operand's strides along the kept / reduced axes (0 where it is broadcast)
};

template <int kOp, int kInput>
__device__ __forceinline__ float term_of(const float *__restrict__ dy, const float *__restrict__ x0,
                                         const float *__restrict__ x1, int64_t iy, int64_t io, float own) {
  if (!reads_inputs<kOp>())
    return grad_of<kOp, kInput>(dy[iy], 0.0f, 0.0f);
  const float other = kInput == 0 ? x1[io] : x0[io];
  return grad_of<kOp, kInput>(dy[iy], kInput == 0 ? own : other, kInput == 0 ? other : own);
}

// Lanes along the operand's innermost kept group (MinMaxInner: ko = outer kept index, w along the contiguous axis,
// reduced index (ro, ri)); block ((ko, tile of tw columns), chunk) takes a run of outer reduced indices, its 256
// threads 256 / tw rows of the tile per step.  The row slots of a column are folded across the lanes, then across the wavefronts, in a
// fixed order; the sums go to partial[(ko * Wk + w) * nchunks + chunk].
template <int kOp, int kInput>
__global__ __launch_bounds__(kBlk) void broadcast2_sum_inner(const float *__restrict__ dy, const float *__restrict__ x0,
                                                             const float *__restrict__ x1, SumAxes Q, MinMaxInner I,
                                                             int nchunks, float *__restrict__ partial) {
  __shared__ float s_part[kBlk / 64][64];
  const MinMaxAxes &A = Q.A;
  const int tw = I.tw, rows_per_step = kBlk / tw;
  const int64_t wtiles = (I.Wk + tw - 1) / tw, ko = blockIdx.x / wtiles, wtile = blockIdx.x - ko * wtiles;
  const int chunk = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cw = tid & (tw - 1), slot = tid / tw;
  const InnerWalk W = inner_walk(dy, A, I, ko, chunk, nchunks);
  const int64_t ybase = W.base - dy;
  const int64_t obase = A.nkept > 1 ? strided_offset(ko, A.nkept - 1, A.ksize, Q.ok) : 0;
  const int64_t ow = Q.ok[A.nkept - 1], ori = Q.orr[A.nred - 1];
  const float *operand = kInput == 0 ? x0 : x1;
  constexpr int kRows = 4;
  {
    const int64_t wcol = wtile * tw + cw;
    const bool col_in = wcol < I.Wk;
    const float own = (reads_inputs<kOp>() && col_in) ? operand[ko * I.Wk + wcol] : 0.0f;
    float acc = 0.0f;
    for (int64_t ro = W.ro_begin; ro < W.ro_end; ++ro) {
      const int64_t oy = ybase + (A.nred > 1 ? strided_offset(ro, A.nred - 1, A.rsize, A.rstride) : 0) + wcol;
      const int64_t oo = obase + (A.nred > 1 ? strided_offset(ro, A.nred - 1, A.rsize, Q.orr) : 0) + wcol * ow;
      for (int64_t ri0 = 0; ri0 < I.Rin; ri0 += kRows * rows_per_step) {
        float t[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const int64_t ri = ri0 + slot + j * rows_per_step;
          t[j] = (col_in && ri < I.Rin) ? term_of<kOp, kInput>(dy, x0, x1, oy + ri * I.rin_stride, oo + ri * ori, own)
                                        : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j)
          acc += t[j];
      }
    }
    for (int off = 32; off >= tw; off >>= 1)
      acc += __shfl_xor(acc, off);
    s_part[wave][lane] = acc;
    __syncthreads();
    if (tid < tw && col_in) {
      float sum = s_part[0][tid];
      for (int w = 1; w < kBlk / 64; ++w)
        sum += s_part[w][tid];
      partial[(ko * I.Wk + wcol) * nchunks + chunk] = sum;
    }
  }
}

// Lanes along the innermost run of terms (MinMaxRows: T lanes per run of Rin contiguous terms, 256 / T kept indices
// per step); block (tile of kept indices, chunk) takes a run of the outer reduced indices.
// Where the kept indices are fewer than the runs a block has in flight (a scalar operand), `vs` of a block's runs
// share a kept index and take every vs-th group of outer reduced indices: vs partial sums per (index, chunk).
// kVec 4: runs that are multiples of four long in 16-byte aligned arrays, four consecutive terms per lane and step
// (the other operand is contiguous along the run or one value for it).
template <int kOp, int kInput, int kVec>
__global__ __launch_bounds__(kBlk) void broadcast2_sum_rows(const float *__restrict__ dy, const float *__restrict__ x0,
                                                            const float *__restrict__ x1, SumAxes Q, MinMaxRows R, int T,
                                                            int vs, int nchunks, float *__restrict__ partial) {
  const MinMaxAxes &A = Q.A;
  const int tid = threadIdx.x, li = tid & (T - 1), slot = tid / T, rps = kBlk / T;
  const int64_t v = (int64_t)blockIdx.x * rps + slot, k = v / vs;
  const int sub = (int)(v - k * vs);
  const bool k_in = k < R.K;
  const int chunk = blockIdx.y;
  const RowWalk W = row_walk(R, chunk, nchunks);
  const int64_t ybase = strided_offset(k_in ? k : 0, A.nkept, A.ksize, A.kstride);
  const int64_t obase = strided_offset(k_in ? k : 0, A.nkept, A.ksize, Q.ok);
  const int64_t ori = Q.orr[A.nred - 1];
  const float *operand = kInput == 0 ? x0 : x1;
  const float *other = kInput == 0 ? x1 : x0;
  const float own = (reads_inputs<kOp>() && k_in) ? operand[k] : 0.0f;
  float acc = 0.0f;
  constexpr int kRows = kVec == 4 ? 4 : 8; // outer reduced indices in flight per lane
  for (int64_t ro = W.ro_begin + (int64_t)sub * kRows; ro < W.ro_end; ro += (int64_t)kRows * vs) {
    int64_t oy[kRows], oo[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j) {
      const bool in = A.nred > 1 && ro + j < W.ro_end;
      oy[j] = ybase + (in ? strided_offset(ro + j, A.nred - 1, A.rsize, A.rstride) : 0);
      oo[j] = obase + (in ? strided_offset(ro + j, A.nred - 1, A.rsize, Q.orr) : 0);
    }
    for (int64_t ri = (int64_t)li * kVec; ri < R.Rin; ri += (int64_t)T * kVec) {
      if (kVec == 4) {
        float4_v gy[kRows], ov[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          const bool in = k_in && ro + j < W.ro_end;
          gy[j] = in ? *reinterpret_cast<const float4_v *>(dy + oy[j] + ri) : float4_v{0.0f, 0.0f, 0.0f, 0.0f};
          if (reads_inputs<kOp>() && in) {
            if (ori)
              ov[j] = *reinterpret_cast<const float4_v *>(other + oo[j] + ri);
            else
              ov[j] = float4_v{other[oo[j]], other[oo[j]], other[oo[j]], other[oo[j]]};
          } else {
            ov[j] = float4_v{1.0f, 1.0f, 1.0f, 1.0f};
          }
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          if (!(k_in && ro + j < W.ro_end))
            continue;
          const float g4[4] = {gy[j].x, gy[j].y, gy[j].z, gy[j].w}, o4[4] = {ov[j].x, ov[j].y, ov[j].z, ov[j].w};
#pragma unroll
          for (int c = 0; c < 4; ++c)
            acc += grad_of<kOp, kInput>(g4[c], kInput == 0 ? own : o4[c], kInput == 0 ? o4[c] : own);
        }
      } else {
        float t[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j)
          t[j] = (k_in && ro + j < W.ro_end) ? term_of<kOp, kInput>(dy, x0, x1, oy[j] + ri, oo[j] + ri * ori, own) : 0.0f;
#pragma unroll
        for (int j = 0; j < kRows; ++j)
          acc += t[j];
      }
    }
  }
  for (int o = T >> 1; o >= 1; o >>= 1)
    acc += __shfl_xor(acc, o);
  if (li == 0 && k_in)
    partial[(k * nchunks + chunk) * vs + sub] = acc;
}

// dx[j] (+)= the partial sums of element j, added in order
__global__ __launch_bounds__(kBlk) void broadcast2_sum_final(const float *__restrict__ partial, int nchunks,
                                                             float *__restrict__ dx, int64_t count, int accum) {
  const int64_t j = (int64_t)blockIdx.x * kBlk + threadIdx.x;
  if (j >= count)
    return;
  float acc = 0.0f;
  for (int c = 0; c < nchunks; ++c)
    acc += partial[j * nchunks + c];
  dx[j] = (accum ? dx[j] : 0.0f) + acc;
}
// ... a wavefront per element where an element has many partial sums
__global__ __launch_bounds__(64) void broadcast2_sum_final_wave(const float *__restrict__ partial, int nchunks,
                                                                float *__restrict__ dx, int accum) {
  const int64_t j = blockIdx.x;
  float acc = 0.0f;
  for (int c = threadIdx.x; c < nchunks; c += 64)
    acc += partial[j * nchunks + c];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    acc += __shfl_xor(acc, off);
  if (threadIdx.x == 0)
    dx[j] = (accum ? dx[j] : 0.0f) + acc;
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

bool reciprocals(const Groups &g, Reciprocals &rc) {
  if (g.total >= ((int64_t)1 << 31))
    return false;
  for (int d = 0; d < g.nd; ++d) {
    const uint64_t n = (uint64_t)g.shape[d];
    int p = 0;
    while (((uint64_t)1 << p) < n)
      ++p;
    rc.shift[d] = 31 + p;
    rc.magic[d] = (uint32_t)((((uint64_t)1 << (31 + p)) / n) + 1);
  }
  return true;
}
// four elements of the innermost group per thread
bool quads(const Groups &g, const void *a, const void *b, const void *c) {
  return g.shape[g.nd - 1] % 4 == 0 && aligned16(a) && aligned16(b) && aligned16(c);
}

template <int kOp> int forward(const float *x0, const float *x1, float *y, const Groups &g, hipStream_t s) {
  Reciprocals rc;
  if (reciprocals(g, rc) && quads(g, x0, x1, y))
    hipLaunchKernelGGL((broadcast2_forward4<kOp>), dim3(blocks_for(g.total / 4)), dim3(kBlk), 0, s, x0, x1, y, g, rc);
  else if (g.total < ((int64_t)1 << 31))
    hipLaunchKernelGGL((broadcast2_forward<kOp, uint32_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, x0, x1, y, g);
  else
    hipLaunchKernelGGL((broadcast2_forward<kOp, int64_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, x0, x1, y, g);
  NBLA_HIP_LAUNCH_CHECK("broadcast2 forward");
  return NBLA_HIP_OK;
}

// The strided sum that forms the gradient of broadcast operand `input`: its axes, which of the two forms it takes
// and into how many partial sums per element.
struct SumPlan {
  bool ok, inner;
  SumAxes Q;
  MinMaxInner I;
  MinMaxRows R;
  int64_t row_chunks;    // row form: blocks per tile of kept indices
  int64_t chunks, count; // (chunks: partial sums per element the workspace holds)
};
SumPlan make_sum_plan(const Groups &g, int input) {
  SumPlan P;
  P.ok = false;
  P.count = g.count[input];
  MinMaxAxes &A = P.Q.A;
  A.nkept = A.nred = 0;
  for (int d = 0; d < g.nd; ++d) {
    if (g.shape[d] == 1)
      continue;
    if (g.s[input][d] != 0) {
      A.ksize[A.nkept] = g.shape[d], A.kstride[A.nkept] = g.sy[d], P.Q.ok[A.nkept++] = g.s[1 - input][d];
    } else {
      A.rsize[A.nred] = g.shape[d], A.rstride[A.nred] = g.sy[d], P.Q.orr[A.nred++] = g.s[1 - input][d];
    }
  }
  if (A.nred == 0)
    return P; // nothing to add up
  if (A.nkept == 0) { // a scalar operand: one kept index
    A.ksize[0] = 1, A.kstride[0] = 0, P.Q.ok[0] = 0;
    A.nkept = 1;
  }
  // one long run of terms (a scalar operand, a bias per sample): cut it into runs of at most 4096 so that the blocks
  // have outer indices to share
  if (A.rstride[A.nred - 1] == 1 && A.nred < 8) {
    const int64_t run = A.rsize[A.nred - 1];
    int64_t piece = 0;
    for (int64_t c = 4096; c >= 64 && run >= 8192; --c)
      if (run % c == 0) {
        piece = c;
        break;
      }
    if (piece) {
      const int64_t so = P.Q.orr[A.nred - 1];
      A.rsize[A.nred] = piece, A.rstride[A.nred] = 1, P.Q.orr[A.nred] = so;
      A.rsize[A.nred - 1] = run / piece, A.rstride[A.nred - 1] = piece, P.Q.orr[A.nred - 1] = so * piece;
      ++A.nred;
    }
  }
  // the operand's innermost group kept: a long run of terms per column under few columns is cut into an outer and an
  // inner part so that the blocks have outer indices to share
  if (A.kstride[A.nkept - 1] == 1 && A.nred < 8) {
    int64_t outer = 1;
    for (int d = 0; d + 1 < A.nred; ++d)
      outer *= A.rsize[d];
    const int64_t run = A.rsize[A.nred - 1], columns = P.count;
    int64_t piece = 0;
    for (int64_t c = 256; c >= 16 && run >= 1024 && outer * columns < 65536; --c)
      if (run % c == 0) {
        piece = c;
        break;
      }
    if (piece) {
      const int64_t sy = A.rstride[A.nred - 1], so = P.Q.orr[A.nred - 1];
      A.rsize[A.nred] = piece, A.rstride[A.nred] = sy, P.Q.orr[A.nred] = so;
      A.rsize[A.nred - 1] = run / piece, A.rstride[A.nred - 1] = sy * piece, P.Q.orr[A.nred - 1] = so * piece;
      ++A.nred;
    }
  }
  P.I = inner_form(A);
  if (P.I.ok) {
    P.inner = true;
    const int64_t tiles = P.I.Ko * ((P.I.Wk + P.I.tw - 1) / P.I.tw);
    P.chunks = (2048 + tiles - 1) / tiles;
    if (P.chunks > P.I.Rout)
      P.chunks = P.I.Rout;
    if (P.chunks > 1024)
      P.chunks = 1024;
    P.ok = tiles <= 0x7fffffffll;
    if (!P.ok)
      return P;
  } else {
    P.R = row_form(A);
    if (!P.R.ok)
      return P;
    P.inner = false;
    // (the lanes per run, and with them the runs a block has in flight, depend on whether the pointers allow 16-byte
    // accesses: the workspace is sized for the form with more partial sums)
    P.row_chunks = row_chunks(P.R);
    int64_t most = 1;
    for (int vec : {1, 4}) {
      const int64_t rps = kBlk / row_lanes(P.R, vec), vs = P.R.K < rps ? rps / P.R.K : 1;
      most = vs > most ? vs : most;
    }
    P.chunks = P.row_chunks * most;
  }
  P.ok = P.count <= 0x7fffffffll;
  return P;
}

template <int kOp, int kInput>
int backward(const float *dy, const float *x0, const float *x1, float *dx, const Groups &g, int accum, void *workspace,
             size_t workspace_bytes, hipStream_t s) {
  if (g.count[kInput] == g.total) {
    Reciprocals rc;
    if (reciprocals(g, rc) && quads(g, dy, dx, dx) && (!reads_inputs<kOp>() || (aligned16(x0) && aligned16(x1))))
      hipLaunchKernelGGL((broadcast2_grad_dense4<kOp, kInput>), dim3(blocks_for(g.total / 4)), dim3(kBlk), 0, s, dy,
                         x0, x1, dx, g, rc, accum);
    else if (g.total < ((int64_t)1 << 31))
      hipLaunchKernelGGL((broadcast2_grad_dense<kOp, kInput, uint32_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, dy,
                         x0, x1, dx, g, accum);
    else
      hipLaunchKernelGGL((broadcast2_grad_dense<kOp, kInput, int64_t>), dim3(blocks_for(g.total)), dim3(kBlk), 0, s, dy,
                         x0, x1, dx, g, accum);
    NBLA_HIP_LAUNCH_CHECK("broadcast2 backward");
    return NBLA_HIP_OK;
  }
  if (g.count[kInput] > 0x7fffffffll)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "broadcast2 backward: a broadcast operand of 2^31 elements or more.");
  const SumPlan P = make_sum_plan(g, kInput);
  if (P.ok && workspace && aligned256(workspace) &&
      workspace_bytes >= (size_t)P.count * P.chunks * sizeof(float)) {
    float *partial = static_cast<float *>(workspace);
    int64_t chunks = P.chunks; // partial sums per element of this launch
    if (P.inner) {
      const int64_t tiles = P.I.Ko * ((P.I.Wk + P.I.tw - 1) / P.I.tw);
      hipLaunchKernelGGL((broadcast2_sum_inner<kOp, kInput>), dim3((unsigned)tiles, (unsigned)P.chunks), dim3(kBlk), 0,
                         s, dy, x0, x1, P.Q, P.I, (int)P.chunks, partial);
    } else {
      const bool vec4 = P.R.Rin % 4 == 0 && aligned16(dy) && (P.Q.orr[P.Q.A.nred - 1] == 0 || P.Q.orr[P.Q.A.nred - 1] == 1) &&
                        (!reads_inputs<kOp>() || (aligned16(x0) && aligned16(x1)));
      const int T = row_lanes(P.R, vec4 ? 4 : 1);
      const int64_t rps = kBlk / T;
      const int vs = P.R.K < rps ? (int)(rps / P.R.K) : 1;
      chunks = P.row_chunks * vs;
      const dim3 grid((unsigned)((P.R.K * vs + rps - 1) / rps), (unsigned)P.row_chunks);
      if (vec4)
        hipLaunchKernelGGL((broadcast2_sum_rows<kOp, kInput, 4>), grid, dim3(kBlk), 0, s, dy, x0, x1, P.Q, P.R, T, vs,
                           (int)P.row_chunks, partial);
      else
        hipLaunchKernelGGL((broadcast2_sum_rows<kOp, kInput, 1>), grid, dim3(kBlk), 0, s, dy, x0, x1, P.Q, P.R, T, vs,
                           (int)P.row_chunks, partial);
    }
    NBLA_HIP_LAUNCH_CHECK("broadcast2 backward sums");
    if (chunks <= 16 && P.count >= 64)
      hipLaunchKernelGGL(broadcast2_sum_final, dim3((unsigned)((P.count + kBlk - 1) / kBlk)), dim3(kBlk), 0, s, partial,
                         (int)chunks, dx, P.count, accum);
    else
      hipLaunchKernelGGL(broadcast2_sum_final_wave, dim3((unsigned)P.count), dim3(64), 0, s, partial, (int)chunks, dx,
                         accum);
    NBLA_HIP_LAUNCH_CHECK("broadcast2 backward");
    return NBLA_HIP_OK;
  }
  hipLaunchKernelGGL((broadcast2_grad_reduce<kOp, kInput>), dim3((unsigned)g.count[kInput]), dim3(kBlk), 0, s, dy, x0,
                     x1, dx, g, accum);
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

size_t nbla_hip_broadcast2_backward_workspace_bytes(int input, const int64_t *shape0, const int64_t *shape1,
                                                    int ndim) {
  Groups g;
  if ((input != 0 && input != 1) || make_groups(g, ndim, shape0, shape1, "broadcast2 backward"))
    return 0;
  if (g.count[input] == g.total || g.count[input] == 0 || g.count[input] > 0x7fffffffll)
    return 0;
  const SumPlan P = make_sum_plan(g, input);
  return P.ok ? round_up((size_t)P.count * P.chunks * sizeof(float), 256) : 0;
}

int nbla_hip_broadcast2_backward_f32(int op, int input, const float *dy, const float *x0, const int64_t *shape0,
                                     const float *x1, const int64_t *shape1, float *dx, int ndim, int accum,
                                     void *workspace, size_t workspace_bytes, void *stream) {
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
  return input == 0 ? backward<OP, 0>(dy, x0, x1, dx, g, accum, workspace, workspace_bytes, s)                         \
                    : backward<OP, 1>(dy, x0, x1, dx, g, accum, workspace, workspace_bytes, s)
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
