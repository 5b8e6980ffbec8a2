// General fp32 product y = (x . w) * colscale + bias on v_mfma_f32_32x32x2_f32:
// the fallback for binary layers whose Sign(W) is not representable as +-1 bits (an arbitrary quantize_zero_to
// with exact zero weights) and the reference product of nbla_hip_affine_f32.  LDS-tiled 128x128x16, four
// wavefronts each owning a 64x64 corner.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 16, kPad = 4;

// w is [K, N] (kTransB == false) or [N, K] (kTransB == true).  Output element (m, n) goes to
// y[(m / inner) * outer_stride + n * n_stride + (m % inner)] (added to what is there with `accumulate`).  `kscale`
// (may be null) scales x along the contraction: x[m, k] * kscale[k] is what gets multiplied (rounded first, as a
// separate scaling pass would).
template <bool kTransB>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                       const float *__restrict__ colscale,
                                                       const float *__restrict__ bias, float *__restrict__ y,
                                                       int64_t M, int64_t K, int64_t N, int64_t inner,
                                                       int64_t outer_stride, int64_t n_stride,
                                                       const int *__restrict__ run_if,
                                                       const float *__restrict__ kscale, int accumulate) {
  if (run_if && *run_if == 0) // uniform over the grid: every block leaves at once
    return;
  __shared__ float As[kBK][kBM + kPad]; // [k][m]
  __shared__ float Bs[kBK][kBN + kPad]; // [k][n]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int64_t m0 = (int64_t)blockIdx.y * kBM, n0 = (int64_t)blockIdx.x * kBN;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  const int a_row = tid >> 1, a_k = (tid & 1) * 8; // 128 rows x 2 halves of 8 k
  const int b_k = tid >> 4, b_n = (tid & 15) * 8;  // [K,N] source: 16 k x 16 groups of 8 n
  const int t_n = tid >> 1, t_k = (tid & 1) * 8;   // [N,K] source: 128 n x 2 halves of 8 k

  for (int64_t k0 = 0; k0 < K; k0 += kBK) {
    float av[8], bv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int64_t m = m0 + a_row, k = k0 + a_k + e;
      av[e] = (m < M && k < K) ? (kscale ? x[m * K + k] * kscale[k] : x[m * K + k]) : 0.0f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (kTransB) {
        const int64_t n = n0 + t_n, k = k0 + t_k + e;
        bv[e] = (k < K && n < N) ? w[n * K + k] : 0.0f;
      } else {
        const int64_t k = k0 + b_k, n = n0 + b_n + e;
        bv[e] = (k < K && n < N) ? w[k * N + n] : 0.0f;
      }
    }
    __syncthreads(); // previous tile fully consumed
#pragma unroll
    for (int e = 0; e < 8; ++e)
      As[a_k + e][a_row] = av[e];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (kTransB)
        Bs[t_k + e][t_n] = bv[e];
      else
        Bs[b_k][b_n + e] = bv[e];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kBK; kk += 2) {
      const int kr = kk + (lane >> 5);
      float af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = As[kr][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[j] = Bs[kr][wn * 64 + j * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  }

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
    if (n >= N)
      continue;
    const float sc = colscale ? colscale[n] : 1.0f;
    const float bi = bias ? bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < M) {
          float v = acc[i][j][r];
          if (colscale)
            v = v * sc;
          if (bias)
            v = v + bi;
          const int64_t off = (inner == 1) ? m * outer_stride : (m / inner) * outer_stride + (m % inner);
          y[off + n * n_stride] = accumulate ? y[off + n * n_stride] + v : v;
        }
      }
  }
}

} // namespace

int launch_gemm_f32_mapped(const float *x, const float *w, bool trans_b, const float *colscale, const float *bias,
                           float *y, int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride,
                           int64_t n_stride, hipStream_t stream, const int *run_if, const float *kscale,
                           bool accumulate) {
  const dim3 grid((unsigned)ceil_div(N, kBN), (unsigned)ceil_div(M, kBM));
  if (trans_b)
    hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, dim3(256), 0, stream, x, w, colscale, bias, y, M, K, N, inner,
                       outer_stride, n_stride, run_if, kscale, accumulate ? 1 : 0);
  else
    hipLaunchKernelGGL(gemm_f32_kernel<false>, grid, dim3(256), 0, stream, x, w, colscale, bias, y, M, K, N, inner,
                       outer_stride, n_stride, run_if, kscale, accumulate ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("gemm_f32");
  return NBLA_HIP_OK;
}

int launch_gemm_f32(const float *x, const float *w, const float *colscale, const float *bias, float *y, int64_t M,
                    int64_t K, int64_t N, hipStream_t stream, const int *run_if) {
  return launch_gemm_f32_mapped(x, w, false, colscale, bias, y, M, K, N, 1, N, 1, stream, run_if, nullptr, false);
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" int nbla_hip_affine_f32(const float *x, const float *w, const float *bias, float *y, int64_t M, int64_t K,
                                   int64_t N, void *stream) {
  if (M <= 0 || K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid GEMM shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  int rc = ensure_init();
  if (rc)
    return rc;
  return launch_gemm_f32(x, w, nullptr, bias, y, M, K, N, as_stream(stream));
}
