// Whole-operation forwards of BinaryWeightAffine / BinaryConnectAffine: weight
// preparation, activation split and the bit-weight product chained on one stream.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

// Rows of x holding a NaN or an infinity cannot be scaled to integers: the digit operand marks them (shift == kBadRow)
// and the matrix-core product leaves NaN in their whole output row.  The reference's product propagates such values
// element by element (affine.cpp:87-95: Inf * w = +-Inf, Inf - Inf = NaN, NaN anywhere = NaN), so those rows -- rare --
// are recomputed as plain fp32 dot products over the materialised weights Wb (* alpha): by the kernel that splits x
// into digits where that kernel is the one-pass form (the product then leaves the rows alone), by this kernel after
// the product otherwise.  Block b looks at rows b, b + gridDim.x, ...
__global__ __launch_bounds__(256) void affine_redo_marked_rows(const float *__restrict__ x, const float *__restrict__ Wb,
                                                               const float *__restrict__ alpha,
                                                               const float *__restrict__ bias, float *__restrict__ y,
                                                               const int32_t *__restrict__ shift, int64_t M, int64_t K,
                                                               int64_t N) {
  for (int64_t m = blockIdx.x; m < M; m += gridDim.x) {
    if (shift[m] != kBadRow) // uniform over the block
      continue;
    for (int64_t n = threadIdx.x; n < N; n += 256) {
      const float a = alpha ? alpha[n] : 1.0f;
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        const float w = alpha ? Wb[k * N + n] * a : Wb[k * N + n]; // the scaled weight the reference multiplies with
        acc = acc + x[m * K + k] * w;
      }
      y[m * N + n] = bias ? acc + bias[n] : acc;
    }
  }
}

struct AffineWorkspace {
  size_t bits_off, split_off, prep_off, count_off, gemm_off, gemm_bytes, total;
};

AffineWorkspace plan_affine(int64_t M, int64_t K, int64_t N) {
  AffineWorkspace w;
  size_t off = 0;
  w.bits_off = off;
  off += round_up(nbla_hip_packed_bits_bytes(K, N), 256);
  w.split_off = off;
  off += round_up(nbla_hip_digit_operand_bytes(M, K), 256);
  w.prep_off = off;
  off += round_up(nbla_hip_binarize_workspace_bytes(K, N), 256);
  w.count_off = off;
  off += 256;
  // partial results of a product whose contraction is spread over the CUs (very small M), or of the one-walk form
  // when it walks K in slices
  w.gemm_off = off;
  w.gemm_bytes = nbla_hip_gemm_bits_workspace_bytes(M, K, N);
  const size_t rows_bytes = round_up(rows_affine_workspace_bytes(M, K, N), 256);
  if (rows_bytes > w.gemm_bytes)
    w.gemm_bytes = rows_bytes;
  off += w.gemm_bytes;
  w.total = off;
  // the one-pass form for very few rows keeps its slab partials at the start of the same buffer
  const size_t small = round_up(small_m_affine_workspace_bytes(M, K, N), 256);
  if (small > w.total)
    w.total = small;
  return w;
}

int binary_affine_forward(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                          int64_t M, int64_t K, int64_t N, float zero_to, void *workspace, size_t workspace_bytes,
                          void *stream_, bool one_walk = false) {
  if (M <= 0 || K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid affine shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  const AffineWorkspace ws = plan_affine(M, K, N);
  if (workspace_bytes < ws.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "binary affine workspace too small (%zu < %zu) or misaligned.", workspace_bytes,
                ws.total);
  char *base = static_cast<char *>(workspace);
  if (one_walk && !rows_affine_covers(W, Wb, alpha, bias, y, M, K, N))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "one-walk binary affine: shape or alignment not covered (M=%lld, K=%lld, "
                "N=%lld).", (long long)M, (long long)K, (long long)N);
  if (!one_walk && small_m_affine_applies(x, W, Wb, alpha, bias, y, M, K, N, zero_to)) {
    const int rc = ensure_init();
    if (rc)
      return rc;
    return launch_small_m_affine(x, W, Wb, alpha, bias, y, M, K, N, zero_to, base, workspace_bytes,
                                 as_stream(stream_));
  }
  uint32_t *bits = reinterpret_cast<uint32_t *>(base + ws.bits_off);
  void *xsplit = base + ws.split_off; // digit operand of x
  void *prep = base + ws.prep_off;
  int *count = reinterpret_cast<int *>(base + ws.count_off);
  // Sign(0) = zero_to that is neither +1 nor -1 cannot be a sign bit: the matrix-core product is then only valid when
  // W holds no weight that is neither negative nor positive.  The kernel that walks W counts such weights on the
  // device; the fp32 product over the materialised signs is launched behind the matrix-core one with that count as
  // its go-ahead and replaces y when it is non-zero (it leaves at once otherwise).  The host never reads the count.
  const bool representable = (zero_to == 1.0f || zero_to == -1.0f);
  hipStream_t stream = as_stream(stream_);
  int rc;

  if (one_walk || (rows_affine_covers(W, Wb, alpha, bias, y, M, K, N) && rows_affine_pays(M, K, N))) {
    // one walk over W: signs, column sums and the product together
    if (!representable && (rc = launch_clear_words(count, 1, stream)))
      return rc;
    if ((rc = launch_split_digits_rows_redo(x, K, nullptr, xsplit, M, K, nullptr, nullptr, stream)))
      return rc;
    if ((rc = launch_rows_affine(xsplit, W, Wb, alpha, bias, y, M, K, N, zero_to, count, base + ws.gemm_off,
                                 ws.gemm_bytes, stream)))
      return rc;
  } else {
    rc = nbla_hip_binarize_weights_f32(W, Wb, alpha, bits, K, N, 0, zero_to, representable ? nullptr : count, prep,
                                       nbla_hip_binarize_workspace_bytes(K, N), stream_);
    if (rc)
      return rc;
    // rows of x with a NaN or an infinity: computed by the splitting kernel where it can, else after the product
    const RowRedo redo{Wb, alpha, bias, y, N};
    bool redone = false;
    rc = launch_split_digits_rows_redo(x, K, nullptr, xsplit, M, K, &redo, &redone, stream);
    if (rc)
      return rc;
    rc = launch_gemm_bits(xsplit, bits, alpha, bias, y, M, K, N, 1, N, 1, false, stream, false, base + ws.gemm_off,
                          ws.gemm_bytes, redone);
    if (rc)
      return rc;
    if (redone)
      return representable ? NBLA_HIP_OK : launch_gemm_f32(x, Wb, alpha, bias, y, M, K, N, stream, count);
  }
  const int32_t *shift =
      reinterpret_cast<const int32_t *>(static_cast<const char *>(xsplit) + digit_operand(M, K).shift_off);
  const unsigned blocks = (unsigned)(M < 256 ? M : 256);
  hipLaunchKernelGGL(affine_redo_marked_rows, dim3(blocks), dim3(256), 0, stream, x, Wb, alpha, bias, y, shift, M, K,
                     N);
  NBLA_HIP_LAUNCH_CHECK("affine_redo_marked_rows");
  return representable ? NBLA_HIP_OK : launch_gemm_f32(x, Wb, alpha, bias, y, M, K, N, stream, count);
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

size_t nbla_hip_binary_affine_workspace_bytes(int64_t M, int64_t K, int64_t N) { return plan_affine(M, K, N).total; }

int nbla_hip_binary_weight_affine_f32(const float *x, const float *W, float *Wb, float *alpha, const float *bias,
                                      float *y, int64_t M, int64_t K, int64_t N, float quantize_zero_to,
                                      void *workspace, size_t workspace_bytes, void *stream) {
  if (!alpha)
    return fail(NBLA_HIP_ERR_VALUE, "BinaryWeightAffine needs an alpha output of size N.");
  return binary_affine_forward(x, W, Wb, alpha, bias, y, M, K, N, quantize_zero_to, workspace, workspace_bytes,
                               stream);
}

int nbla_hip_binary_affine_one_walk_f32(const float *x, const float *W, float *Wb, float *alpha, const float *bias,
                                        float *y, int64_t M, int64_t K, int64_t N, float quantize_zero_to,
                                        void *workspace, size_t workspace_bytes, void *stream) {
  return binary_affine_forward(x, W, Wb, alpha, bias, y, M, K, N, quantize_zero_to, workspace, workspace_bytes, stream,
                               true);
}

int nbla_hip_binary_connect_affine_f32(const float *x, const float *W, float *Wb, const float *bias, float *y,
                                       int64_t M, int64_t K, int64_t N, float quantize_zero_to, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  return binary_affine_forward(x, W, Wb, nullptr, bias, y, M, K, N, quantize_zero_to, workspace, workspace_bytes,
                               stream);
}

} // extern "C"
