// y = x . W (+ b) for a handful of rows of x and real-valued weights: with at most 16 rows the product is a single
// pass over W, and turning W into digit operands for the matrix cores costs several such passes.  Plain fp32 on the
// vector units, the contraction in ascending k inside a slab of K and the slabs added in order (affine.cpp:87-95 adds
// in Eigen's order: equal to rounding; NaN and Inf propagate element by element as there).
//
// Block (1024 columns, slab of K): a thread owns four consecutive columns (one 16-byte load per row of W, eight rows
// in flight), the slab's rows of x sit in LDS and are read as broadcast 16-byte words (four k per read); a thread
// keeps kM x 4 sums.  The slabs' partial results [slab][m][n] are added by a second launch, which adds the bias.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

constexpr int kFewBlock = 256;
typedef float float4_f __attribute__((ext_vector_type(4)));

template <int kM>
__global__ __launch_bounds__(kFewBlock) void affine_few_rows(const float *__restrict__ x, const float *__restrict__ W,
                                                             float *__restrict__ partial, int M, int64_t K, int64_t N,
                                                             int64_t slab_k) {
  extern __shared__ __attribute__((aligned(16))) float s_x[]; // [kM][slab_k]
  const int tid = threadIdx.x;
  const int64_t k0 = (int64_t)blockIdx.y * slab_k, k1 = k0 + slab_k < K ? k0 + slab_k : K;
  const int64_t n0 = ((int64_t)blockIdx.x * kFewBlock + tid) * 4;
  for (int64_t i = tid; i < (int64_t)kM * slab_k; i += kFewBlock) {
    const int64_t m = i / slab_k, k = k0 + (i - m * slab_k);
    s_x[i] = (m < M && k < k1) ? x[m * K + k] : 0.0f;
  }
  __syncthreads();
  const bool col_in = n0 < N; // (N is a multiple of four)
  const float *wp = W + (col_in ? n0 : 0);
  float acc[kM][4];
#pragma unroll
  for (int m = 0; m < kM; ++m)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      acc[m][c] = 0.0f;
  constexpr int kBatch = 8; // rows of W in flight per thread
  for (int64_t kb = k0; kb < k1; kb += kBatch) {
    float4_f w[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      // (rows past the slab count as zeros: their x is zero too, and 0 * 0 adds nothing whatever W holds elsewhere)
      w[j] = kb + j < k1 ? *reinterpret_cast<const float4_f *>(wp + (kb + j) * N) : float4_f{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int j4 = 0; j4 < kBatch; j4 += 4) {
#pragma unroll
      for (int m = 0; m < kM; ++m) {
        const float4_f xv = *reinterpret_cast<const float4_f *>(s_x + (int64_t)m * slab_k + (kb - k0) + j4);
        const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          acc[m][0] = acc[m][0] + xs[u] * w[j4 + u].x;
          acc[m][1] = acc[m][1] + xs[u] * w[j4 + u].y;
          acc[m][2] = acc[m][2] + xs[u] * w[j4 + u].z;
          acc[m][3] = acc[m][3] + xs[u] * w[j4 + u].w;
        }
      }
    }
  }
  if (col_in) {
#pragma unroll
    for (int m = 0; m < kM; ++m)
      if (m < M)
        *reinterpret_cast<float4_f *>(partial + ((int64_t)blockIdx.y * M + m) * N + n0) =
            float4_f{acc[m][0], acc[m][1], acc[m][2], acc[m][3]};
  }
}

__global__ __launch_bounds__(kFewBlock) void affine_few_rows_finish(const float *__restrict__ partial, int slabs,
                                                                    const float *__restrict__ bias,
                                                                    float *__restrict__ y, int64_t MN, int64_t N) {
  const int64_t i = (int64_t)blockIdx.x * kFewBlock + threadIdx.x;
  if (i >= MN)
    return;
  float acc = partial[i];
  for (int s = 1; s < slabs; ++s)
    acc = acc + partial[(int64_t)s * MN + i];
  y[i] = bias ? acc + bias[i % N] : acc;
}

struct FewRowsPlan {
  int64_t slab_k;
  int slabs, rows; // rows: the kernel's row count (a power of two covering M)
};
FewRowsPlan few_rows_plan(int64_t M, int64_t K, int64_t N) {
  FewRowsPlan p;
  p.rows = 1;
  while (p.rows < M)
    p.rows *= 2;
  const int64_t col_blocks = ceil_div(N, (int64_t)kFewBlock * 4);
  int64_t slabs = ceil_div(768, col_blocks);
  // the partial results are written and read once: keep them to a quarter of W's bytes
  const int64_t by_traffic = K / (8 * M) > 0 ? K / (8 * M) : 1;
  if (slabs > by_traffic)
    slabs = by_traffic;
  // a slab of x in LDS: at most 32 KiB, a multiple of eight rows of W
  int64_t slab_k = ceil_div(ceil_div(K, slabs), 8) * 8;
  const int64_t lds_k = (8192 / p.rows) / 8 * 8;
  if (slab_k > lds_k)
    slab_k = lds_k;
  p.slab_k = slab_k;
  p.slabs = (int)ceil_div(K, slab_k);
  return p;
}

} // namespace

bool affine_few_rows_applies(const float *x, const float *W, const float *y, int64_t M, int64_t K, int64_t N) {
  return M >= 1 && M <= 16 && N % 4 == 0 && N >= 4 && K >= 1 && aligned16(W) && aligned16(y) && x != nullptr &&
         K * N >= ((int64_t)1 << 20); // (small products are bound by their launches either way)
}
size_t affine_few_rows_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M < 1 || M > 16 || K < 1 || N < 1)
    return 0;
  const FewRowsPlan p = few_rows_plan(M, K, N);
  return round_up((size_t)p.slabs * M * N * sizeof(float), 256);
}
int launch_affine_few_rows(const float *x, const float *W, const float *bias, float *y, int64_t M, int64_t K, int64_t N,
                           void *workspace, size_t workspace_bytes, hipStream_t stream) {
  const FewRowsPlan p = few_rows_plan(M, K, N);
  if (workspace_bytes < (size_t)p.slabs * M * N * sizeof(float) || !aligned16(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "affine (few rows): workspace too small or misaligned.");
  float *partial = static_cast<float *>(workspace);
  const dim3 grid((unsigned)ceil_div(N, (int64_t)kFewBlock * 4), (unsigned)p.slabs);
  const size_t lds = (size_t)p.rows * p.slab_k * sizeof(float);
#define NBLA_FEW_ROWS(R)                                                                                               \
  hipLaunchKernelGGL(affine_few_rows<R>, grid, dim3(kFewBlock), lds, stream, x, W, partial, (int)M, K, N, p.slab_k)
  switch (p.rows) {
  case 1: NBLA_FEW_ROWS(1); break;
  case 2: NBLA_FEW_ROWS(2); break;
  case 4: NBLA_FEW_ROWS(4); break;
  case 8: NBLA_FEW_ROWS(8); break;
  default: NBLA_FEW_ROWS(16); break;
  }
#undef NBLA_FEW_ROWS
  NBLA_HIP_LAUNCH_CHECK("affine_few_rows");
  const int64_t MN = M * N;
  hipLaunchKernelGGL(affine_few_rows_finish, dim3((unsigned)ceil_div(MN, kFewBlock)), dim3(kFewBlock), 0, stream,
                     partial, p.slabs, bias, y, MN, N);
  NBLA_HIP_LAUNCH_CHECK("affine_few_rows_finish");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
