// Outputs of a digit x digit product that a NaN or an infinity reaches, recomputed one by one.
//
// The digit operands mark a row that holds a non-finite value (shift == kBadRow) and the product leaves NaN in every
// output of a marked row of either operand.  The reference's products propagate such values output by output
// (affine.cpp:87-95, convolution.cpp:185-193: Inf * w = +-Inf, Inf - Inf = NaN, 0 * Inf = NaN, a finite row times
// finite weights stays finite), so those outputs -- rare -- are recomputed here as plain fp32 dot products in
// ascending k, then + bias.
#pragma once
#include "common.hpp"
#include "conv_geom.hpp"
#include "gemm_layout.hpp"

namespace nbla_hip {

// Element (m, k) of the left operand: a dense row-major matrix, or the unfolded input of a convolution group.
struct DenseRows {
  const float *x;
  int64_t K;
  __device__ __forceinline__ float operator()(int64_t m, int64_t k) const { return x[m * K + k]; }
};
struct UnfoldedRows {
  const float *x;
  ConvGeom g;
  int64_t grp;
  __device__ __forceinline__ float operator()(int64_t m, int64_t k) const { return col_value(x, g, grp, m, k); }
};

// y[m, n] = sum_k rows(m, k) * W[k * w_k_stride + n * w_n_stride] (+ bias[n]) for every m with shift_a[m] == kBadRow
// and every n with shift_b[n] == kBadRow; y[m, n] sits at (m / inner) * outer_stride + m % inner + n * n_stride.  A
// block looks at 256 marks at a time and moves on at once when none of them is set.
template <class Rows>
__global__ __launch_bounds__(256) void product_redo_marked(Rows rows, const float *__restrict__ W, int64_t w_k_stride,
                                                           int64_t w_n_stride, const float *__restrict__ bias,
                                                           float *__restrict__ y, int64_t inner, int64_t outer_stride,
                                                           int64_t n_stride, const int32_t *__restrict__ shift_a,
                                                           const int32_t *__restrict__ shift_b, int64_t M, int64_t K,
                                                           int64_t N) {
  auto element = [&](int64_t m, int64_t n) {
    float acc = 0.0f;
    for (int64_t k = 0; k < K; ++k)
      acc = acc + rows(m, k) * W[k * w_k_stride + n * w_n_stride];
    const int64_t q = m / inner;
    y[q * outer_stride + (m - q * inner) + n * n_stride] = bias ? acc + bias[n] : acc;
  };
  for (int64_t base = (int64_t)blockIdx.x * 256; base < M; base += (int64_t)gridDim.x * 256) {
    const int64_t mine = base + threadIdx.x;
    if (!__syncthreads_or(mine < M && shift_a[mine] == kBadRow))
      continue;
    const int64_t end = base + 256 < M ? base + 256 : M;
    for (int64_t m = base; m < end; ++m)
      if (shift_a[m] == kBadRow) // uniform over the block
        for (int64_t n = threadIdx.x; n < N; n += 256)
          element(m, n);
  }
  for (int64_t base = (int64_t)blockIdx.x * 256; base < N; base += (int64_t)gridDim.x * 256) {
    const int64_t mine = base + threadIdx.x;
    if (!__syncthreads_or(mine < N && shift_b[mine] == kBadRow))
      continue;
    const int64_t end = base + 256 < N ? base + 256 : N;
    for (int64_t n = base; n < end; ++n)
      if (shift_b[n] == kBadRow) // uniform over the block
        for (int64_t m = threadIdx.x; m < M; m += 256)
          if (shift_a[m] != kBadRow) // (those rows are done)
            element(m, n);
  }
}

// a_digits / b_digits: the two digit operands of the product that has just been launched on `stream` (their shift
// arrays are the marks).
template <class Rows>
int launch_product_redo(const Rows &rows, const float *W, int64_t w_k_stride, int64_t w_n_stride, const float *bias,
                        float *y, int64_t inner, int64_t outer_stride, int64_t n_stride, const void *a_digits,
                        const void *b_digits, int64_t M, int64_t K, int64_t N, hipStream_t stream) {
  const int32_t *shift_a =
      reinterpret_cast<const int32_t *>(static_cast<const char *>(a_digits) + digit_operand(M, K).shift_off);
  const int32_t *shift_b =
      reinterpret_cast<const int32_t *>(static_cast<const char *>(b_digits) + digit_operand(N, K).shift_off);
  int64_t blocks = ceil_div(M > N ? M : N, 256);
  if (blocks > 1024)
    blocks = 1024;
  hipLaunchKernelGGL(product_redo_marked<Rows>, dim3((unsigned)blocks), dim3(256), 0, stream, rows, W, w_k_stride,
                     w_n_stride, bias, y, inner, outer_stride, n_stride, shift_a, shift_b, M, K, N);
  NBLA_HIP_LAUNCH_CHECK("product_redo_marked");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
