// Backward passes of the affine products: BinaryWeightAffine / BinaryConnectAffine (gradient w.r.t. x on the
// bit-weight product) and Affine with real-valued weights (INQAffine), plus the bias gradient.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"
#include "redo_marked.hpp"

namespace nbla_hip {
namespace {

// Column sums (bias gradients) in a fixed order: slices of `rows` rows (256, or 64 when that leaves fewer than a
// thousand blocks), inside a slice four interleaved row groups per column, folded through LDS in group order; then
// the slices in slice order.
constexpr int kSumCols = 64;
inline int column_sum_rows(int64_t M, int64_t N) {
  return ceil_div(N, kSumCols) * ceil_div(M, 256) >= 1024 ? 256 : 64;
}

// partial[s][n] = sum of dy[m][n] over the rows m of slice s; block = 64 columns x 4 row groups.
__global__ __launch_bounds__(256) void column_sum_partial(const float *__restrict__ dy, float *__restrict__ partial,
                                                          int64_t M, int64_t N, int rows) {
  __shared__ float part[4][kSumCols];
  const int c = threadIdx.x & (kSumCols - 1), rg = threadIdx.x >> 6;
  const int64_t n = (int64_t)blockIdx.x * kSumCols + c;
  const int64_t m0 = (int64_t)blockIdx.y * rows, m1 = (m0 + rows < M) ? m0 + rows : M;
  float acc = 0.0f;
  if (n < N) {
#pragma unroll 8
    for (int64_t m = m0 + rg; m < m1; m += 4)
      acc += dy[m * N + n];
  }
  part[rg][c] = acc;
  __syncthreads();
  if (rg == 0 && n < N)
    partial[(int64_t)blockIdx.y * N + n] = ((part[0][c] + part[1][c]) + part[2][c]) + part[3][c];
}

__global__ __launch_bounds__(256) void column_sum_final(const float *__restrict__ partial, float *__restrict__ db,
                                                        int64_t slices, int64_t N, int accumulate) {
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= N)
    return;
  float acc = 0.0f;
#pragma unroll 8
  for (int64_t s = 0; s < slices; ++s)
    acc += partial[s * N + n];
  db[n] = accumulate ? db[n] + acc : acc;
}

struct BackwardPlan {
  size_t bits_off, digits_off, prep_off, count_off, a_planes_off, b_planes_off, flag_off, sums_off, split_off,
      split_bytes, total;
};

// One layout for all three backward entry points (the regions a call does not use are simply left alone).
BackwardPlan plan_backward(int64_t M, int64_t K, int64_t N) {
  BackwardPlan p;
  size_t off = 0;
  p.bits_off = off; // packed Sign(W) with the roles of k and n exchanged
  off += round_up(nbla_hip_packed_bits_bytes(N, K), 256);
  p.digits_off = off; // digit operand of dy (* alpha), M x N
  off += round_up(nbla_hip_digit_operand_bytes(M, N), 256);
  p.prep_off = off;
  off += round_up(nbla_hip_binarize_workspace_bytes(N, K), 256);
  p.count_off = off;
  off += 256;
  // digit operands of x^T and dy^T for dW, and of dy and W for the real-weight dx, share two regions
  const size_t a3 = nbla_hip_digit_operand_bytes(K, M), b3 = nbla_hip_digit_operand_bytes(N, M);
  const size_t a4 = nbla_hip_digit_operand_bytes(M, N), b4 = nbla_hip_digit_operand_bytes(K, N);
  p.a_planes_off = off;
  off += round_up(a3 > a4 ? a3 : a4, 256);
  p.b_planes_off = off;
  off += round_up(b3 > b4 ? b3 : b4, 256);
  p.flag_off = off;
  off += 256;
  p.sums_off = off;
  off += round_up(column_sums_workspace_bytes(M, N), 256);
  p.split_off = off; // partial results of a digit product whose contraction is spread over the CUs (small outputs)
  const size_t s1 = gemm_digits_split_bytes(K, M, N), s2 = gemm_digits_split_bytes(M, N, K);
  p.split_bytes = s1 > s2 ? s1 : s2;
  off += round_up(p.split_bytes, 256);
  p.total = off;
  return p;
}

// dW[K, N] (+)= x^T . dy on the digit x digit product (both factors are real numbers): the operand rows are the
// columns of x and of dy, the contraction runs over the M samples.
int grad_weights(const float *x, const float *dy, float *dW, int64_t M, int64_t K, int64_t N, bool accumulate,
                 char *base, const BackwardPlan &p, hipStream_t stream) {
  int rc = launch_split_digits_columns(x, K, base + p.a_planes_off, M, K, false, stream);
  if (rc)
    return rc;
  rc = launch_split_digits_columns(dy, N, base + p.b_planes_off, M, N, false, stream);
  if (rc)
    return rc;
  return launch_gemm_digits(base + p.a_planes_off, base + p.b_planes_off, nullptr, dW, K, M, N, 1, N, 1, stream,
                            accumulate, base + p.split_off, p.split_bytes);
}

// dx[M, K] (+)= dy' . W^T with real-valued weights, dy' [M, N], on the digit x digit product: both operands are
// row-scaled (rows m of dy', rows k of W, contraction over n)
int grad_input_planes(const float *dyp, const float *W, float *dx, int64_t M, int64_t K, int64_t N, bool accumulate,
                      char *base, const BackwardPlan &p, hipStream_t stream) {
  int rc = nbla_hip_split_digits_f32(dyp, N, base + p.a_planes_off, M, N, stream);
  if (rc)
    return rc;
  rc = nbla_hip_split_digits_f32(W, N, base + p.b_planes_off, K, N, stream);
  if (rc)
    return rc;
  return launch_gemm_digits(base + p.a_planes_off, base + p.b_planes_off, nullptr, dx, M, N, K, 1, K, 1, stream,
                            accumulate, base + p.split_off, p.split_bytes);
}

int check_args(int64_t M, int64_t K, int64_t N, void *workspace, size_t workspace_bytes, const BackwardPlan &p) {
  if (M <= 0 || K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid affine shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  if (workspace_bytes < p.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "affine backward workspace too small (%zu < %zu) or misaligned.", workspace_bytes,
                p.total);
  return ensure_init();
}

} // namespace

size_t column_sums_workspace_bytes(int64_t M, int64_t N) { return (size_t)ceil_div(M, 64) * N * sizeof(float); }

int launch_column_sums(const float *dy, float *db, int64_t M, int64_t N, bool accumulate, void *partial,
                       hipStream_t stream) {
  const int rows = column_sum_rows(M, N);
  const int64_t slices = ceil_div(M, rows);
  hipLaunchKernelGGL(column_sum_partial, dim3((unsigned)ceil_div(N, kSumCols), (unsigned)slices), dim3(256), 0, stream,
                     dy, static_cast<float *>(partial), M, N, rows);
  NBLA_HIP_LAUNCH_CHECK("column_sum_partial");
  hipLaunchKernelGGL(column_sum_final, dim3((unsigned)ceil_div(N, 256)), dim3(256), 0, stream,
                     static_cast<const float *>(partial), db, slices, N, accumulate ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("column_sum_final");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

size_t nbla_hip_affine_backward_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M <= 0 || K <= 0 || N <= 0)
    return 0;
  return plan_backward(M, K, N).total;
}

int nbla_hip_binary_affine_backward_f32(const float *dy, const float *x, const float *W, const float *Wb,
                                        const float *alpha, float *dx, float *dW, float *db, int64_t M, int64_t K,
                                        int64_t N, float quantize_zero_to, int accum_x, int accum_w, int accum_b,
                                        void *workspace, size_t workspace_bytes, void *stream_) {
  const BackwardPlan p = plan_backward(M, K, N);
  int rc = check_args(M, K, N, workspace, workspace_bytes, p);
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  char *base = static_cast<char *>(workspace);
  if (dx) {
    const bool representable = (quantize_zero_to == 1.0f || quantize_zero_to == -1.0f);
    uint32_t *bits = reinterpret_cast<uint32_t *>(base + p.bits_off);
    int *count = reinterpret_cast<int *>(base + p.count_off);
    // Sign(W) packed for the contraction over n: W is stored [K, N] = [output column of dx][contraction]
    rc = nbla_hip_binarize_weights_f32(W, nullptr, nullptr, bits, N, K, 1, quantize_zero_to,
                                       representable ? nullptr : count, base + p.prep_off,
                                       nbla_hip_binarize_workspace_bytes(N, K), stream_);
    if (rc)
      return rc;
    // Sign(0) = quantize_zero_to that is neither +1 nor -1 cannot be a sign bit: the pass above has counted, on the
    // device, the weights that are neither negative nor positive.  The matrix-core product does nothing when that
    // count is non-zero, and an fp32 product over the forward's signs Wb, launched behind it, does nothing when it is
    // zero: exactly one of the two writes dx, and the host never reads the count.
    rc = nbla_hip_split_digits_scaled_f32(dy, N, alpha, base + p.digits_off, M, N, stream_);
    if (rc)
      return rc;
    rc = launch_gemm_bits(base + p.digits_off, bits, nullptr, nullptr, dx, M, N, K, 1, K, 1, false, stream,
                          accum_x != 0, nullptr, 0, false, representable ? nullptr : count);
    if (rc)
      return rc;
    if (!representable) {
      if (!Wb)
        return fail(NBLA_HIP_ERR_VALUE, "the binarised weights are needed when Sign(0) is neither +1 nor -1.");
      // dx[m, k] (+)= sum_n (dy[m, n] alpha[n]) Wb[k, n]
      rc = launch_gemm_f32_mapped(dy, Wb, true, nullptr, nullptr, dx, M, N, K, 1, K, 1, stream, count, alpha,
                                  accum_x != 0);
      if (rc)
        return rc;
    }
  }
  if (dW) {
    rc = grad_weights(x, dy, dW, M, K, N, accum_w != 0, base, p, stream);
    if (rc)
      return rc;
  }
  if (db)
    return launch_column_sums(dy, db, M, N, accum_b != 0, base + p.sums_off, stream);
  return NBLA_HIP_OK;
}

int nbla_hip_affine_backward_f32(const float *dy, const float *x, const float *W, float *dx, float *dW, float *db,
                                 int64_t M, int64_t K, int64_t N, int accum_x, int accum_w, int accum_b,
                                 void *workspace, size_t workspace_bytes, void *stream_) {
  const BackwardPlan p = plan_backward(M, K, N);
  int rc = check_args(M, K, N, workspace, workspace_bytes, p);
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  char *base = static_cast<char *>(workspace);
  if (dx) {
    rc = grad_input_planes(dy, W, dx, M, K, N, accum_x != 0, base, p, stream);
    if (rc)
      return rc;
  }
  if (dW) {
    rc = grad_weights(x, dy, dW, M, K, N, accum_w != 0, base, p, stream);
    if (rc)
      return rc;
  }
  if (db)
    return launch_column_sums(dy, db, M, N, accum_b != 0, base + p.sums_off, stream);
  return NBLA_HIP_OK;
}

size_t nbla_hip_affine_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M <= 0 || K <= 0 || N <= 0)
    return 0;
  // the two digit operands, then the partial results of a contraction spread over the CUs (small outputs)
  return round_up(nbla_hip_digit_operand_bytes(M, K), 256) + round_up(nbla_hip_digit_operand_bytes(N, K), 256) +
         round_up(gemm_digits_split_bytes(M, K, N), 256);
}

int nbla_hip_affine_digits_f32(const float *x, const float *W, const float *bias, float *y, int64_t M, int64_t K,
                               int64_t N, void *workspace, size_t workspace_bytes, void *stream_) {
  if (M <= 0 || K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid affine shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  if (workspace_bytes < nbla_hip_affine_workspace_bytes(M, K, N) || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "affine workspace too small or misaligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  // a handful of rows: one fp32 pass over W instead of its conversion to digit operands
  if (affine_few_rows_applies(x, W, y, M, K, N) && workspace_bytes >= affine_few_rows_workspace_bytes(M, K, N))
    return launch_affine_few_rows(x, W, bias, y, M, K, N, workspace, workspace_bytes, stream);
  char *xd = static_cast<char *>(workspace);
  char *wd = xd + round_up(nbla_hip_digit_operand_bytes(M, K), 256);
  rc = nbla_hip_split_digits_f32(x, K, xd, M, K, stream_);
  if (rc)
    return rc;
  rc = launch_split_digits_columns(W, N, wd, K, N, true, stream);
  if (rc)
    return rc;
  char *split = wd + round_up(nbla_hip_digit_operand_bytes(N, K), 256);
  rc = launch_gemm_digits(xd, wd, bias, y, M, K, N, 1, N, 1, stream, false, split, gemm_digits_split_bytes(M, K, N));
  if (rc)
    return rc;
  // rows of x and columns of W holding a NaN or an infinity: their outputs one by one, as affine.cpp:87-95 gives them
  return launch_product_redo(DenseRows{x, K}, W, N, 1, bias, y, 1, N, 1, xd, wd, M, K, N, stream);
}

} // extern "C"
