// y = (x . B) * alpha + bias for sign-binarised weights B, on the gfx950 matrix
// cores.  x arrives as three bf16 planes (x == hi + mid + lo exactly) in MFMA
// fragment order, B as one bit per weight.  Every product (bf16 plane element
// times +-1) is exact, and v_mfma_f32_32x32x16_bf16 accumulates in fp32, so the
// result carries fp32 accumulation error only ("bf16x3" fp32-faithful product).
//
// Work decomposition: a block of kWavesM x kWavesN wavefronts owns a
// BM x BN output tile and walks K in steps of 32.  Per step it stages
//   A: BM/32 row blocks x (2 k blocks x 3 planes) fragments = BM/32 * 6 KiB
//   B: BN/64 column groups x 64 packed words               = BN * 4 B
// from HBM/L2 into LDS through registers (double-buffered, one barrier per
// step).  A fragments are read back with one conflict-free 128-bit LDS load per
// lane; the packed words are expanded to +-1.0 bf16 pairs in registers with two
// VALU operations per register (shift, and-or).
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct GemmBitsArgs {
  const uint4_t *xs;    // split operand
  const uint32_t *bits; // packed weights
  const float *alpha;   // may be null
  const float *bias;    // may be null
  float *y;
  int64_t M, N;
  int64_t row_blocks; // of the split operand
  int64_t k_blocks;   // fragments along k (2 per k step)
  int64_t col_groups; // of the packed operand
  int64_t k_steps;
  int64_t blocks_m, blocks_n;
  int64_t inner, outer_stride, n_stride; // output addressing
};

// Blocks are handed to the 8 XCDs round-robin; give each XCD a contiguous run
// of tiles (n fastest) so that blocks resident on one XCD share an A panel in
// that XCD's L2.
__device__ __forceinline__ int64_t xcd_remap(int64_t b, int64_t total) {
  constexpr int64_t kXcds = 8;
  const int64_t per = total / kXcds, rem = total % kXcds;
  const int64_t xcd = b % kXcds, slot = b / kXcds;
  // XCDs [0, rem) own per+1 tiles, the rest own per tiles.
  const int64_t start = xcd * per + (xcd < rem ? xcd : rem);
  return start + slot;
}

// kSwap exchanges the MFMA operand roles (the instruction computes the transposed 32x32 tile), which puts
// consecutive m on consecutive lanes of the accumulator: the store pattern for outputs whose m index is contiguous.
template <int BM, int BN, int kWavesM, int kWavesN, bool kSwap>
__global__ __launch_bounds__(kWavesM *kWavesN * 64) void gemm_bits_kernel(GemmBitsArgs a) {
  constexpr int kThreads = kWavesM * kWavesN * 64;
  constexpr int MF = BM / kWavesM / 32;  // A fragments per wavefront (rows)
  constexpr int NF = BN / kWavesN / 32;  // B fragments per wavefront (columns)
  constexpr int NW = NF / 2;             // packed words per lane per k step
  static_assert(NF % 2 == 0, "a packed word serves two column fragments");
  constexpr int kASegs = BM / 32;        // row blocks per tile
  constexpr int kASegVec = 6 * 64;       // uint4 per row block per k step (2 k blocks x 3 planes)
  constexpr int kAVec = kASegs * kASegVec;
  constexpr int kAPasses = (kAVec + kThreads - 1) / kThreads;
  constexpr int kBWords = BN;            // BN/64 groups x 64 words
  constexpr int kBPasses = (kBWords + kThreads - 1) / kThreads;
  constexpr int kStageBytes = kAVec * 16 + kBWords * 4;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % kWavesM, wn = wave / kWavesM;

  const int64_t tile = xcd_remap(blockIdx.x, a.blocks_m * a.blocks_n);
  const int64_t bm = tile / a.blocks_n, bn = tile - bm * a.blocks_n;

  // Per-thread source pointers of the global -> LDS copy (constant over k but for
  // a fixed advance per step).  Row blocks / column groups past the end of the
  // operand are clamped: their products land in rows/columns that are not stored.
  const uint4_t *a_src[kAPasses];
#pragma unroll
  for (int p = 0; p < kAPasses; ++p) {
    const int idx = p * kThreads + tid;
    const int seg = idx / kASegVec, within = idx - seg * kASegVec;
    int64_t rb = bm * kASegs + seg;
    if (rb >= a.row_blocks)
      rb = a.row_blocks - 1;
    a_src[p] = a.xs + rb * a.k_blocks * 192 + within;
  }
  const uint32_t *b_src[kBPasses];
#pragma unroll
  for (int p = 0; p < kBPasses; ++p) {
    const int idx = p * kThreads + tid;
    int64_t cg = bn * (BN / 64) + idx / 64;
    if (cg >= a.col_groups)
      cg = a.col_groups - 1;
    b_src[p] = a.bits + cg * 64 + (idx & 63);
  }

  uint4_t a_reg[kAPasses];
  uint32_t b_reg[kBPasses];

  auto load_step = [&](int64_t ks) {
#pragma unroll
    for (int p = 0; p < kAPasses; ++p)
      if (kAVec % kThreads == 0 || p * kThreads + tid < kAVec)
        a_reg[p] = a_src[p][ks * kASegVec];
#pragma unroll
    for (int p = 0; p < kBPasses; ++p)
      if (kBWords % kThreads == 0 || p * kThreads + tid < kBWords)
        b_reg[p] = b_src[p][ks * a.col_groups * 64];
  };
  auto store_step = [&](int buf) {
    uint4_t *sa = reinterpret_cast<uint4_t *>(smem + buf * kStageBytes);
    uint32_t *sb = reinterpret_cast<uint32_t *>(smem + buf * kStageBytes + kAVec * 16);
#pragma unroll
    for (int p = 0; p < kAPasses; ++p)
      if (kAVec % kThreads == 0 || p * kThreads + tid < kAVec)
        sa[p * kThreads + tid] = a_reg[p];
#pragma unroll
    for (int p = 0; p < kBPasses; ++p)
      if (kBWords % kThreads == 0 || p * kThreads + tid < kBWords)
        sb[p * kThreads + tid] = b_reg[p];
  };

  f32x16_t acc[MF][NF];
#pragma unroll
  for (int i = 0; i < MF; ++i)
#pragma unroll
    for (int j = 0; j < NF; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  // Fragment fetch and the MFMA block of one k16 sub-step (s = 0, 1) of a staged tile.
  auto read_a = [&](int buf, int s, uint4_t (&af)[MF][3]) {
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + buf * kStageBytes);
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int p = 0; p < 3; ++p)
        af[i][p] = sa[(wm * MF + i) * kASegVec + s * 192 + p * 64 + lane];
  };
  auto read_words = [&](int buf, uint32_t (&words)[NW]) {
    const uint32_t *sb = reinterpret_cast<const uint32_t *>(smem + buf * kStageBytes + kAVec * 16);
#pragma unroll
    for (int w = 0; w < NW; ++w)
      words[w] = sb[(wn * NW + w) * 64 + lane];
  };
  // Bits -> +-1.0 bf16 pairs: register i of fragment (f, s) is ((word << 4*(2f+s)+i) & 0x80008000) | 0x3F803F80.
  // The two constants are kept in registers so that each register costs a shift and one v_and_or_b32.
  uint32_t sign_mask = 0x80008000u, one_pair = 0x3F803F80u;
  asm volatile("" : "+s"(sign_mask));
  asm volatile("" : "+v"(one_pair));
  auto expand = [&](int s, const uint32_t (&words)[NW], uint4_t (&bf)[NF]) {
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      const uint32_t w = words[j >> 1];
      const int base = 4 * (2 * (j & 1) + s);
      bf[j].x = ((w << (base + 0)) & sign_mask) | one_pair;
      bf[j].y = ((w << (base + 1)) & sign_mask) | one_pair;
      bf[j].z = ((w << (base + 2)) & sign_mask) | one_pair;
      bf[j].w = ((w << (base + 3)) & sign_mask) | one_pair;
    }
  };
  auto mma = [&](const uint4_t (&af)[MF][3], const uint4_t (&bf)[NF]) {
    // smallest plane first: the low-order parts enter the accumulator before the leading one
#pragma unroll
    for (int p = 2; p >= 0; --p)
#pragma unroll
      for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int j = 0; j < NF; ++j) {
          acc[i][j] = kSwap ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[j]),
                                                                      __builtin_bit_cast(bf16x8_t, af[i][p]),
                                                                      acc[i][j], 0, 0, 0)
                            : __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i][p]),
                                                                      __builtin_bit_cast(bf16x8_t, bf[j]),
                                                                      acc[i][j], 0, 0, 0);
        }
  };
  // Asks the scheduler to issue the region just written as: one MFMA, then a few VALU / memory instructions in
  // its shadow, repeated.  A wavefront issues in order and an MFMA occupies the matrix pipe for 32 cycles, so the
  // expansion, fragment fetch and staging traffic of the next sub-step fit between consecutive MFMAs instead of
  // in front of them (where wavefronts running in lockstep would all leave the matrix pipe idle together).
  constexpr int kMfma = 3 * MF * NF;
  constexpr int kValuPer = (NF * 8 + 8 + kMfma - 1) / kMfma + 1;
  auto interleave_first = [&]() { // region: LDS reads of sub-step 1, expansion, MFMAs of sub-step 0, LDS staging writes
#pragma unroll
    for (int g = 0; g < kMfma; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
      if (g < MF * 3)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
      __builtin_amdgcn_sched_group_barrier(0x002, kValuPer, 0); // VALU
      if (g >= kMfma - kAPasses - kBPasses)
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // DS write
    }
  };
  auto interleave_second = [&]() { // region: global loads, LDS reads of the next stage, expansion, MFMAs of sub-step 1
#pragma unroll
    for (int g = 0; g < kMfma; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
      if (g < kAPasses + kBPasses)
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
      if (g < MF * 3 + NW)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
      __builtin_amdgcn_sched_group_barrier(0x002, kValuPer, 0); // VALU
    }
  };

  // Software pipeline.  Two LDS stages, one barrier per k step, no branches in the loop body (the last iterations
  // re-load the final stage instead of skipping, so each half of the body is one scheduling region).  While the
  // MFMA block of one k16 sub-step runs, the A fragments of the next sub-step are fetched from LDS and its B
  // fragments are expanded; the global loads of stage ks+2 are issued a full step ahead of their use.
  uint4_t af0[MF][3], af1[MF][3], bf0[NF], bf1[NF];
  uint32_t wcur[NW], wnext[NW];
  const int64_t last = a.k_steps - 1;
  load_step(0);
  store_step(0);
  __syncthreads();
  load_step(last < 1 ? last : 1);
  read_words(0, wcur);
  read_a(0, 0, af0);
  expand(0, wcur, bf0);
  for (int64_t ks = 0; ks <= last; ++ks) {
    const int buf = (int)(ks & 1);
    // sub-step 0 runs; sub-step 1 is prepared; the staged registers (stage ks+1) go to the other LDS buffer
    read_a(buf, 1, af1);
    expand(1, wcur, bf1);
    mma(af0, bf0);
    store_step(buf ^ 1);
    interleave_first();
    __syncthreads();
    // sub-step 1 runs; global loads of stage ks+2 are issued; sub-step 0 of stage ks+1 is prepared
    load_step(ks + 2 < last ? ks + 2 : last);
    read_words(buf ^ 1, wnext);
    read_a(buf ^ 1, 0, af0);
    expand(0, wnext, bf0);
    mma(af1, bf1);
    interleave_second();
#pragma unroll
    for (int w = 0; w < NW; ++w)
      wcur[w] = wnext[w];
  }

  // Epilogue.  Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
  // column l%32 of the 32x32 fragment; rows are m and columns n, or the reverse
  // under kSwap.
  const int col_in_frag = lane & 31, row_half = lane >> 5;
  if (!kSwap) {
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      const int64_t n = bn * BN + (wn * NF + j) * 32 + col_in_frag;
      if (n >= a.N)
        continue;
      const float al = a.alpha ? a.alpha[n] : 1.0f;
      const float bi = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
      for (int i = 0; i < MF; ++i) {
        const int64_t m0 = bm * BM + (wm * MF + i) * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t m = m0 + 8 * (r >> 2) + 4 * row_half + (r & 3);
          if (m < a.M) {
            float v = acc[i][j][r];
            if (a.alpha)
              v = v * al;
            if (a.bias)
              v = v + bi;
            const int64_t off = (a.inner == 1) ? m * a.outer_stride : (m / a.inner) * a.outer_stride + (m % a.inner);
            a.y[off + n * a.n_stride] = v;
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < MF; ++i) {
      const int64_t m = bm * BM + (wm * MF + i) * 32 + col_in_frag;
      if (m >= a.M)
        continue;
      const int64_t off = (a.inner == 1) ? m * a.outer_stride : (m / a.inner) * a.outer_stride + (m % a.inner);
#pragma unroll
      for (int j = 0; j < NF; ++j) {
        const int64_t n0 = bn * BN + (wn * NF + j) * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t n = n0 + 8 * (r >> 2) + 4 * row_half + (r & 3);
          if (n < a.N) {
            float v = acc[i][j][r];
            if (a.alpha)
              v = v * a.alpha[n];
            if (a.bias)
              v = v + a.bias[n];
            a.y[off + n * a.n_stride] = v;
          }
        }
      }
    }
  }
}

template <int BM, int BN, int kWavesM, int kWavesN, bool kSwap>
int launch_tile(const GemmBitsArgs &args, hipStream_t stream) {
  constexpr int kThreads = kWavesM * kWavesN * 64;
  constexpr int kStageBytes = (BM / 32) * 6 * 64 * 16 + BN * 4;
  constexpr int kSmem = 2 * kStageBytes;
  auto kernel = gemm_bits_kernel<BM, BN, kWavesM, kWavesN, kSwap>;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
    if (e != hipSuccess)
      return fail_hip(e, "hipFuncSetAttribute(gemm_bits LDS size)");
    configured = true;
  }
  GemmBitsArgs a = args;
  a.blocks_m = ceil_div(a.M, BM);
  a.blocks_n = ceil_div(a.N, BN);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(a.blocks_m * a.blocks_n)), dim3(kThreads), kSmem, stream, a);
  NBLA_HIP_LAUNCH_CHECK("gemm_bits");
  return NBLA_HIP_OK;
}

// Tile choice by M (measured on MI355X at K = 4096, N = 11008): the wide 128x512 tile with sixteen wavefronts
// wins once there are enough row blocks to fill the 256 CUs; smaller tiles keep more blocks in flight below that.
template <bool kSwap> int dispatch(const GemmBitsArgs &a, hipStream_t stream) {
  if (a.M >= 3072)
    return launch_tile<128, 512, 4, 4, kSwap>(a, stream);
  if (a.M > 1024)
    return launch_tile<128, 256, 2, 4, kSwap>(a, stream);
  if (a.M > 32)
    return launch_tile<64, 256, 2, 4, kSwap>(a, stream);
  return launch_tile<32, 256, 1, 4, kSwap>(a, stream);
}

} // namespace

int launch_gemm_bits(const void *xsplit, const uint32_t *bits, const float *alpha, const float *bias, float *y,
                     int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride, int64_t n_stride,
                     bool swap_out, hipStream_t stream) {
  if (M <= 0 || K <= 0 || N <= 0 || inner <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid GEMM shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  if (!aligned16(xsplit) || !aligned16(bits))
    return fail(NBLA_HIP_ERR_MEMORY, "GEMM operands must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  GemmBitsArgs a;
  a.xs = static_cast<const uint4_t *>(xsplit);
  a.bits = bits;
  a.alpha = alpha;
  a.bias = bias;
  a.y = y;
  a.M = M;
  a.N = N;
  a.row_blocks = split_row_blocks(M);
  a.k_blocks = split_k_blocks(K);
  a.col_groups = bits_col_groups(N);
  a.k_steps = bits_k_tiles(K);
  a.blocks_m = a.blocks_n = 0;
  a.inner = inner;
  a.outer_stride = outer_stride;
  a.n_stride = n_stride;
  return swap_out ? dispatch<true>(a, stream) : dispatch<false>(a, stream);
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" int nbla_hip_gemm_bits_f32(const void *xsplit, const uint32_t *bits, const float *alpha, const float *bias,
                                      float *y, int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride,
                                      int64_t n_stride, void *stream) {
  // m-contiguous outputs (n_stride != 1) store from the transposed accumulator tile
  return launch_gemm_bits(xsplit, bits, alpha, bias, y, M, K, N, inner, outer_stride, n_stride, n_stride != 1,
                          as_stream(stream));
}
