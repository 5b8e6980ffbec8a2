// fp32-faithful product of two fp32 matrices on the bf16 matrix cores.
// Both operands arrive as bf16 planes in MFMA fragment order:
//   x = xh + xm + xl (exact),  w = wh + wm + wl (exact).
// When every weight is exactly representable in bf16 (INQ weights: zero or a
// signed power of two) only wh is non-zero and three products give the exact
// fp32-accumulated result; otherwise the six leading cross terms are summed
// (xh.wh + xm.wh + xh.wm + xl.wh + xm.wm + xh.wl; the dropped terms are below
// 2^-24 relative).  Which of the two runs is decided on the device from a flag
// written by the kernel that produced the weight planes, so the host never has to
// look at the weights.
//
// Tiling: 128 x 128 output tile per block of four wavefronts (2 x 2, 64 x 64
// each), K in steps of 32, operands staged through LDS with register prefetch.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct GemmPlanesArgs {
  const uint4_t *xs; // [row_blocks][k_blocks][3][64] uint4
  const uint4_t *ws; // [col_blocks][k_blocks][3][64] uint4
  const int *need_low_planes; // device flag: non-zero when wm / wl carry data
  const float *colscale, *bias;
  float *y;
  int64_t M, N, row_blocks, col_blocks, k_blocks, k_steps, blocks_m, blocks_n;
  int64_t inner, outer_stride, n_stride;
  int accumulate; // add to y instead of overwriting it
};

constexpr int kBM = 128, kBN = 128, kThreads = 256;
constexpr int kSegs = 4;           // 32-row (or 32-column) blocks per tile side
constexpr int kSegVec = 6 * 64;    // uint4 per block per k step, all three planes
constexpr int kAVec = kSegs * kSegVec;
constexpr int kAStageBytes = kAVec * 16;

template <int NB>
__device__ __forceinline__ void run_tile(const GemmPlanesArgs &a, unsigned char *smem, f32x16_t (&acc)[2][2], int64_t bm,
                                         int64_t bn) {
  constexpr int kBVec = kSegs * 2 * NB * 64; // uint4 of B per stage
  constexpr int kStageBytes = kAStageBytes + kBVec * 16;
  constexpr int kAPasses = kAVec / kThreads;       // 6
  constexpr int kBPasses = kBVec / kThreads;       // 2 or 6
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;

  const uint4_t *a_src[kAPasses];
#pragma unroll
  for (int p = 0; p < kAPasses; ++p) {
    const int idx = p * kThreads + tid;
    const int seg = idx / kSegVec, within = idx - seg * kSegVec;
    int64_t rb = bm * kSegs + seg;
    if (rb >= a.row_blocks)
      rb = a.row_blocks - 1;
    a_src[p] = a.xs + rb * a.k_blocks * 192 + within;
  }
  const uint4_t *b_src[kBPasses];
#pragma unroll
  for (int p = 0; p < kBPasses; ++p) {
    const int idx = p * kThreads + tid;
    const int seg = idx / (2 * NB * 64);
    const int r = idx - seg * (2 * NB * 64);
    const int s = r / (NB * 64), q = r - s * (NB * 64); // q = plane * 64 + lane
    int64_t cb = bn * kSegs + seg;
    if (cb >= a.col_blocks)
      cb = a.col_blocks - 1;
    b_src[p] = a.ws + cb * a.k_blocks * 192 + s * 192 + q;
  }
  uint4_t a_reg[kAPasses], b_reg[kBPasses];
  auto load_step = [&](int64_t ks) {
#pragma unroll
    for (int p = 0; p < kAPasses; ++p)
      a_reg[p] = a_src[p][ks * kSegVec];
#pragma unroll
    for (int p = 0; p < kBPasses; ++p)
      b_reg[p] = b_src[p][ks * kSegVec];
  };
  auto store_step = [&](int buf) {
    uint4_t *sa = reinterpret_cast<uint4_t *>(smem + buf * kStageBytes);
    uint4_t *sb = reinterpret_cast<uint4_t *>(smem + buf * kStageBytes + kAStageBytes);
#pragma unroll
    for (int p = 0; p < kAPasses; ++p)
      sa[p * kThreads + tid] = a_reg[p];
#pragma unroll
    for (int p = 0; p < kBPasses; ++p)
      sb[p * kThreads + tid] = b_reg[p];
  };

  load_step(0);
  store_step(0);
  __syncthreads();
  for (int64_t ks = 0; ks < a.k_steps; ++ks) {
    const int buf = (int)(ks & 1);
    if (ks + 1 < a.k_steps)
      load_step(ks + 1);
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + buf * kStageBytes);
    const uint4_t *sb = reinterpret_cast<const uint4_t *>(smem + buf * kStageBytes + kAStageBytes);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      uint4_t af[2][3], bf[2][NB];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int p = 0; p < 3; ++p)
          af[i][p] = sa[(wm * 2 + i) * kSegVec + s * 192 + p * 64 + lane];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int p = 0; p < NB; ++p)
          bf[j][p] = sb[((wn * 2 + j) * 2 + s) * (NB * 64) + p * 64 + lane];
      // plane pairs (x plane, w plane), smallest contributions first
      constexpr int kPairs = (NB == 3) ? 6 : 3;
      constexpr int pa[6] = {2, 1, 0, 1, 0, 0};
      constexpr int pb3[6] = {0, 1, 2, 0, 1, 0};
      constexpr int pa1[3] = {2, 1, 0};
#pragma unroll
      for (int t = 0; t < kPairs; ++t) {
        const int xa = (NB == 3) ? pa[t] : pa1[t];
        const int wb = (NB == 3) ? pb3[t] : 0;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i][xa]),
                                                                __builtin_bit_cast(bf16x8_t, bf[j][wb]), acc[i][j], 0,
                                                                0, 0);
      }
    }
    if (ks + 1 < a.k_steps)
      store_step(buf ^ 1);
    __syncthreads();
  }
}

__global__ __launch_bounds__(kThreads) void gemm_planes_kernel(GemmPlanesArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  // one block per CU (98 KiB of LDS): the 32 blocks resident on an XCD cover 4 x 8 tiles
  int64_t bm, bn;
  band_tile<4>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn);
  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;
  if (*a.need_low_planes) // uniform over the grid
    run_tile<3>(a, smem, acc, bm, bn);
  else
    run_tile<1>(a, smem, acc, bm, bn);

  const int col_in_frag = lane & 31, row_half = lane >> 5;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = bn * kBN + (wn * 2 + j) * 32 + col_in_frag;
    if (n >= a.N)
      continue;
    const float sc = a.colscale ? a.colscale[n] : 1.0f;
    const float bi = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t m0 = bm * kBM + (wm * 2 + i) * 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + 8 * (r >> 2) + 4 * row_half + (r & 3);
        if (m < a.M) {
          float v = acc[i][j][r];
          if (a.colscale)
            v = v * sc;
          if (a.bias)
            v = v + bi;
          const int64_t off = (a.inner == 1) ? m * a.outer_stride : (m / a.inner) * a.outer_stride + (m % a.inner);
          if (a.accumulate)
            v = a.y[off + n * a.n_stride] + v;
          a.y[off + n * a.n_stride] = v;
        }
      }
    }
  }
}

__device__ __forceinline__ uint32_t bf16_rne(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Weight planes: one wavefront per (column block, k block) fragment; lane l holds
// column cb*32 + l%32 and k = kb*16 + (l/32)*8 + 0..7.  transposed: w stored [N, K].
__global__ __launch_bounds__(256) void split_weights(const float *__restrict__ w, uint4_t *__restrict__ out,
                                                     int *__restrict__ need_low, int64_t K, int64_t N, int transposed,
                                                     int64_t k_blocks, int64_t frags) {
  const int64_t frag = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (frag >= frags)
    return;
  const int lane = threadIdx.x & 63;
  const int64_t cb = frag / k_blocks, kb = frag - cb * k_blocks;
  const int64_t n = cb * kFragRows + (lane & 31);
  const int64_t k0 = kb * kFragK + (lane >> 5) * 8;
  uint32_t h[8], mi[8], l[8];
  uint32_t low = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t k = k0 + e;
    const float v = (n < N && k < K) ? (transposed ? w[n * K + k] : w[k * N + n]) : 0.0f;
    const uint32_t u = __float_as_uint(v);
    if ((u & 0x7f800000u) == 0x7f800000u) {
      h[e] = (u >> 16) | ((u & 0xffffu) ? 0x40u : 0u);
      mi[e] = l[e] = 0u;
    } else {
      h[e] = bf16_rne(v);
      if ((h[e] & 0x7f80u) == 0x7f80u)
        h[e] = u >> 16;
      const float r1 = v - __uint_as_float(h[e] << 16);
      mi[e] = bf16_rne(r1);
      const float r2 = r1 - __uint_as_float(mi[e] << 16);
      l[e] = bf16_rne(r2);
    }
    low |= (mi[e] & 0x7fffu) | (l[e] & 0x7fffu);
  }
  uint4_t o;
  uint4_t *dst = out + frag * 3 * 64 + lane;
  o.x = h[0] | (h[1] << 16), o.y = h[2] | (h[3] << 16), o.z = h[4] | (h[5] << 16), o.w = h[6] | (h[7] << 16);
  dst[0] = o;
  o.x = mi[0] | (mi[1] << 16), o.y = mi[2] | (mi[3] << 16), o.z = mi[4] | (mi[5] << 16), o.w = mi[6] | (mi[7] << 16);
  dst[64] = o;
  o.x = l[0] | (l[1] << 16), o.y = l[2] | (l[3] << 16), o.z = l[4] | (l[5] << 16), o.w = l[6] | (l[7] << 16);
  dst[128] = o;
  // one flag for the whole grid: look before writing, or millions of wavefronts queue on one address
  if (__any(low != 0) && lane == 0 && __hip_atomic_load(need_low, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
    atomicOr(need_low, 1);
}

__global__ void clear_flag(int *flag) { *flag = 0; }

} // namespace

int launch_split_weights(const float *w, void *planes, int *need_low, int64_t K, int64_t N, bool transposed,
                         hipStream_t stream) {
  const int64_t k_blocks = split_k_blocks(K);
  const int64_t frags = split_row_blocks(N) * k_blocks;
  hipLaunchKernelGGL(clear_flag, dim3(1), dim3(1), 0, stream, need_low);
  hipLaunchKernelGGL(split_weights, dim3((unsigned)ceil_div(frags, 4)), dim3(256), 0, stream, w,
                     static_cast<uint4_t *>(planes), need_low, K, N, transposed ? 1 : 0, k_blocks, frags);
  NBLA_HIP_LAUNCH_CHECK("split_weights");
  return NBLA_HIP_OK;
}

int launch_gemm_planes(const void *xsplit, const void *wplanes, const int *need_low, const float *colscale,
                       const float *bias, float *y, int64_t M, int64_t K, int64_t N, int64_t inner,
                       int64_t outer_stride, int64_t n_stride, hipStream_t stream, bool accumulate) {
  constexpr int kSmem = 2 * (kAStageBytes + kSegs * 2 * 3 * 64 * 16);
  static std::atomic<uint64_t> configured{0};
  const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(gemm_planes_kernel), kSmem, configured,
                                       "hipFuncSetAttribute(gemm_planes LDS size)");
  if (rc_lds)
    return rc_lds;
  GemmPlanesArgs a;
  a.xs = static_cast<const uint4_t *>(xsplit);
  a.ws = static_cast<const uint4_t *>(wplanes);
  a.need_low_planes = need_low;
  a.colscale = colscale;
  a.bias = bias;
  a.y = y;
  a.M = M;
  a.N = N;
  a.row_blocks = split_row_blocks(M);
  a.col_blocks = split_row_blocks(N);
  a.k_blocks = split_k_blocks(K);
  a.k_steps = bits_k_tiles(K);
  a.blocks_m = ceil_div(M, kBM);
  a.blocks_n = ceil_div(N, kBN);
  a.inner = inner;
  a.outer_stride = outer_stride;
  a.n_stride = n_stride;
  a.accumulate = accumulate ? 1 : 0;
  hipLaunchKernelGGL(gemm_planes_kernel, dim3((unsigned)(a.blocks_m * a.blocks_n)), dim3(kThreads), kSmem, stream, a);
  NBLA_HIP_LAUNCH_CHECK("gemm_planes");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
