// BinaryWeightAffine / BinaryConnectAffine forward for a handful of input rows (M <= 64), in ONE pass over W.
// Two forms: dot products on the vector ALUs (this comment; up to 16 rows), and on the matrix cores (second half of
// the file; 9 to 64 rows).
//
// With so few rows the product is bound by the weights: 4 B read and 4 B written (the fp32 signs Wb are an output of
// the function) per weight, against 2 M flop.  The general path walks W once to binarise it and then runs the packed
// bits through the matrix cores in further launches; here the same walk that writes Sign(W) and sums |W| per column
// also forms the dot products, on the vector ALUs: every weight a thread has in registers is turned into its sign s
// and added to  acc[m] += s * x[m, k]  for each of the M rows.  W is read in 1 KiB runs (a wavefront covers 256
// consecutive columns of a row) with a second batch of rows in flight while the first is consumed.
//
// The rows of x are the same for every lane: they are fetched with scalar loads and never occupy vector registers.
//
// Work decomposition: block = kWavesK wavefronts stacked in K; wavefront wk walks kRowsPerWave rows of the block's
// 256-column strip.  The block's wavefronts fold their accumulators over wk through LDS (fixed order), and the block writes one
// partial row per input row, plus the |W| column sums, for its slab of K.  A second, tiny launch adds the slabs in
// slab order, forms alpha = colsum * ((float)1 / K) and scales: y = (sum_k s * x) * alpha + bias.  Every sum runs in a
// fixed order, so results do not change from run to run.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

#include <string.h>

namespace nbla_hip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));

// Four wavefronts stacked in K over one 256-column strip; four such blocks per CU (128 registers per lane), so the
// whole of a 4096 x 11008 weight matrix (688 blocks) is resident at once and no second round of blocks trails behind.
constexpr int kWavesK = 4, kWavesN = 1;
constexpr int kThreads = 64 * kWavesK * kWavesN;
constexpr int blocks_per_cu(int MT) { return MT >= 16 ? 2 : 4; } // sixteen rows need more than 128 registers
constexpr int kRowsPerWave = 64;                     // rows of W one wavefront walks
constexpr int kSlabRows = kWavesK * kRowsPerWave;    // rows of W per block
constexpr int kWaveCols = 256;                       // 64 lanes x float4
constexpr int kStripCols = kWavesN * kWaveCols;      // columns per block

// sign.hpp:48-50: w > 0 ? 1 : (w < 0 ? -1 : zero_to).  +-0 and NaN are exactly the inputs that are neither less nor
// greater than zero; every other input takes 1 with its own sign bit.
__device__ __forceinline__ float sign_of(float w, float zero_to) {
  const float one = __uint_as_float((__float_as_uint(w) & 0x80000000u) | 0x3f800000u);
  return __builtin_islessgreater(w, 0.0f) ? one : zero_to;
}

__host__ __device__ inline int64_t small_m_slabs(int64_t K) { return ceil_div(K, kSlabRows); }
__host__ __device__ inline int64_t small_m_padded_cols(int64_t N) { return ceil_div(N, kStripCols) * kStripCols; }

// partial[slab][r][Npad]: r < MT the dot products of input row r over the slab, r == MT the |W| column sums.
//
// The activations never enter vector registers: x[m, k] is the same for every lane, so it is read with scalar loads
// and enters the multiply-add as a scalar operand.  kFull (decided per block) is the interior of W, where no row or
// column test is needed; edge blocks run the same code with clamped loads and guarded stores.
template <int MT, int kBatch, bool kFull>
__device__ __forceinline__ void small_m_walk(const float *__restrict__ W, float *__restrict__ Wb,
                                             const float *__restrict__ x, int64_t M, int64_t K, int64_t N,
                                             int64_t k_wave, int64_t n0, float zero_to, float (&acc)[MT][4],
                                             float (&cs)[4]) {
  constexpr int kBatches = kRowsPerWave / kBatch;
  static_assert(kBatches % 2 == 0, "the loop below consumes two batches per trip");
  constexpr int kXRows = (32 / MT) < 1 ? 1 : ((32 / MT) > kBatch ? kBatch : (32 / MT)); // rows whose x is fetched at once
  const bool col_ok = kFull || n0 < N;
  const int64_t n_ld = col_ok ? n0 : N - 4; // loads are unconditional: a clamped address, masked afterwards
  const uint32_t lane_bytes = (uint32_t)(n_ld * 4);
  float4_t va[kBatch], vb[kBatch];
  auto load_batch = [&](int b, float4_t (&dst)[kBatch]) {
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      int64_t k = k_wave + b * kBatch + j;
      if (!kFull && k >= K)
        k = K - 1;
      const char *row = reinterpret_cast<const char *>(W + k * N); // uniform base + 32-bit lane offset
      // ordinary loads, nontemporal stores: the combination that streams fastest here (nontemporal loads cost a fifth)
      dst[j] = *reinterpret_cast<const float4_t *>(row + lane_bytes);
    }
  };
  auto consume_batch = [&](int b, const float4_t (&src)[kBatch]) {
#pragma unroll
    for (int j0 = 0; j0 < kBatch; j0 += kXRows) {
      float xv[kXRows][MT];
#pragma unroll
      for (int jj = 0; jj < kXRows; ++jj)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const int64_t k = k_wave + b * kBatch + j0 + jj;
          const bool ok = m < M && (kFull || k < K); // uniform
          xv[jj][m] = ok ? x[(int64_t)m * K + k] : 0.0f;
        }
#pragma unroll
      for (int jj = 0; jj < kXRows; ++jj) {
        const int j = j0 + jj;
        const int64_t k = k_wave + b * kBatch + j;
        float4_t w = src[j];
        if (!kFull && k >= K)
          w = float4_t{0.0f, 0.0f, 0.0f, 0.0f}; // |0| adds nothing, and the row's x reads as zero
        float s[4];
        s[0] = sign_of(w.x, zero_to), s[1] = sign_of(w.y, zero_to);
        s[2] = sign_of(w.z, zero_to), s[3] = sign_of(w.w, zero_to);
        if (kFull || (col_ok && k < K)) {
          float4_t o;
          o.x = s[0], o.y = s[1], o.z = s[2], o.w = s[3];
          char *row = reinterpret_cast<char *>(Wb + k * N);
          __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(row + lane_bytes));
        }
        cs[0] += fabsf(w.x), cs[1] += fabsf(w.y), cs[2] += fabsf(w.z), cs[3] += fabsf(w.w);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            acc[m][c] = __builtin_fmaf(s[c], xv[jj][m], acc[m][c]);
      }
    }
  };
  // Two batches of rows are in registers at any time: one being consumed, one in flight.  The loop is kept rolled
  // so that the compiler does not hoist further batches (their registers would spill).
  load_batch(0, va);
#pragma clang loop unroll(disable)
  for (int b = 0; b < kBatches; b += 2) {
    load_batch(b + 1, vb);
    consume_batch(b, va);
    if (b + 2 < kBatches)
      load_batch(b + 2, va);
    consume_batch(b + 1, vb);
  }
}

template <int MT, int kBatch>
__global__ __launch_bounds__(kThreads, blocks_per_cu(MT)) void binary_affine_small_m(const float *__restrict__ W, float *__restrict__ Wb,
                                                                  const float *__restrict__ x,
                                                                  float *__restrict__ partial, int64_t M, int64_t K,
                                                                  int64_t N, int64_t Npad, float zero_to) {
  constexpr int kVals = (MT + 1) * 4; // accumulators per lane
  __shared__ __attribute__((aligned(16))) float red[2 * kWavesN * kVals * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform: row indices stay in scalar registers
  const int wn = wave % kWavesN, wk = wave / kWavesN;
  const int64_t slab = blockIdx.y;
  const int64_t k_slab = slab * kSlabRows;
  const int64_t n0 = (int64_t)blockIdx.x * kStripCols + wn * kWaveCols + 4 * lane;
  const int64_t k_wave = k_slab + wk * kRowsPerWave;

  float acc[MT][4];
  float cs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      acc[m][c] = 0.0f;

  const bool full = k_slab + kSlabRows <= K && ((int64_t)blockIdx.x + 1) * kStripCols <= N && M == MT;
  if (full)
    small_m_walk<MT, kBatch, true>(W, Wb, x, M, K, N, k_wave, n0, zero_to, acc, cs);
  else
    small_m_walk<MT, kBatch, false>(W, Wb, x, M, K, N, k_wave, n0, zero_to, acc, cs);

  // Fold over wk in a fixed order: (wk0 + wk2) + (wk1 + wk3), through LDS.
  auto slot = [&](int s) { return red + ((size_t)(s * kWavesN + wn) * kVals) * 64 + lane; };
  auto put = [&](float *dst) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        dst[(m * 4 + c) * 64] = acc[m][c];
#pragma unroll
    for (int c = 0; c < 4; ++c)
      dst[(MT * 4 + c) * 64] = cs[c];
  };
  auto add = [&](const float *src) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        acc[m][c] += src[(m * 4 + c) * 64];
#pragma unroll
    for (int c = 0; c < 4; ++c)
      cs[c] += src[(MT * 4 + c) * 64];
  };
  if (wk >= 2)
    put(slot(wk - 2));
  __syncthreads();
  if (wk < 2)
    add(slot(wk));
  __syncthreads();
  if (wk == 1)
    put(slot(1));
  __syncthreads();
  if (wk != 0)
    return;
  add(slot(1));
  float *out = partial + (size_t)slab * (MT + 1) * Npad + n0; // n0 < Npad always
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    float4_t o;
    o.x = acc[m][0], o.y = acc[m][1], o.z = acc[m][2], o.w = acc[m][3];
    *reinterpret_cast<float4_t *>(out + (size_t)m * Npad) = o;
  }
  float4_t o;
  o.x = cs[0], o.y = cs[1], o.z = cs[2], o.w = cs[3];
  *reinterpret_cast<float4_t *>(out + (size_t)MT * Npad) = o;
}

// Thread (m, four columns): the slabs in slab order, alpha (binary_weight_affine.cpp:68: the column sum times the
// rounded reciprocal of K), scale, bias.
template <int MT>
__global__ __launch_bounds__(256) void binary_affine_small_m_finish(const float *__restrict__ partial,
                                                                    float *__restrict__ alpha,
                                                                    const float *__restrict__ bias,
                                                                    float *__restrict__ y, int64_t M, int64_t N,
                                                                    int64_t Npad, int64_t slabs, float inv_k) {
  const int64_t n0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const int m = blockIdx.y;
  if (n0 >= N)
    return;
  float4_t dot = {0.0f, 0.0f, 0.0f, 0.0f}, cs = {0.0f, 0.0f, 0.0f, 0.0f};
  // eight slabs' loads are issued before the first is added (the adds keep slab order)
  constexpr int kAhead = 8;
  const size_t slab_stride = (size_t)(MT + 1) * Npad;
  for (int64_t s0 = 0; s0 < slabs; s0 += kAhead) {
    float4_t d[kAhead], c[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int64_t s = (s0 + j < slabs) ? s0 + j : slabs - 1; // clamped loads, masked below
      const float *p = partial + (size_t)s * slab_stride + n0;
      d[j] = *reinterpret_cast<const float4_t *>(p + (size_t)m * Npad);
      if (alpha)
        c[j] = *reinterpret_cast<const float4_t *>(p + (size_t)MT * Npad);
    }
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      if (s0 + j >= slabs)
        break;
      dot.x += d[j].x, dot.y += d[j].y, dot.z += d[j].z, dot.w += d[j].w;
      if (alpha)
        cs.x += c[j].x, cs.y += c[j].y, cs.z += c[j].z, cs.w += c[j].w;
    }
  }
  if (alpha) {
    float4_t a;
    a.x = cs.x * inv_k, a.y = cs.y * inv_k, a.z = cs.z * inv_k, a.w = cs.w * inv_k;
    if (m == 0)
      *reinterpret_cast<float4_t *>(alpha + n0) = a;
    dot.x = dot.x * a.x, dot.y = dot.y * a.y, dot.z = dot.z * a.z, dot.w = dot.w * a.w;
  }
  if (bias) {
    const float4_t b = *reinterpret_cast<const float4_t *>(bias + n0);
    dot.x = dot.x + b.x, dot.y = dot.y + b.y, dot.z = dot.z + b.z, dot.w = dot.w + b.w;
  }
  *reinterpret_cast<float4_t *>(y + (size_t)m * N + n0) = dot;
}

template <int MT, int kBatch>
int launch_small_m(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y, int64_t M,
                   int64_t K, int64_t N, float zero_to, float *partial, hipStream_t stream) {
  const int64_t Npad = small_m_padded_cols(N), slabs = small_m_slabs(K);
  hipLaunchKernelGGL((binary_affine_small_m<MT, kBatch>), dim3((unsigned)(Npad / kStripCols), (unsigned)slabs),
                     dim3(kThreads), 0, stream, W, Wb, x, partial, M, K, N, Npad, zero_to);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_small_m");
  hipLaunchKernelGGL(binary_affine_small_m_finish<MT>, dim3((unsigned)ceil_div(N / 4, 256), (unsigned)M), dim3(256), 0,
                     stream, partial, alpha, bias, y, M, N, Npad, slabs, (float)1 / K);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_small_m_finish");
  return NBLA_HIP_OK;
}


// ---------------------------------------------------------------------------------------------------------------
// Seventeen to sixty-four input rows: the same single walk over W, with the dot products on the matrix cores.
//
// The vector-ALU form above spends one multiply-add per weight and input row, which no longer hides behind the
// weight stream past sixteen rows.  Here a wavefront turns every 16 x 128 tile of W into the B operands of
// v_mfma_f32_32x32x16_bf16 as it passes through the registers: lane (h, c) = (lane / 32, lane % 32) loads the float4
// of rows 8h .. 8h+7 at columns 4c .. 4c+3, so for each of the four column offsets j the lane holds exactly what
// the instruction wants from it for "column c" of a 16 x 32 operand: eight consecutive k.  The sign of a weight as
// bf16 is the upper half of its fp32 sign (+-1, or zero_to), one byte permute per pair.  Product j yields the output
// columns 4c + j, so a lane ends up with float4 runs of the output as well.
// The A operand is x itself, split exactly into three bf16 terms (8 + 8 + 8 significand bits: x = hi + mid + lo, each
// the truncation of what the previous ones left), so every product sign x term is exact and the sums are
// accumulated in fp32 by the instruction.  Inf and NaN stay in the first term (the remainders of a non-finite value
// are dropped), which makes them spread per output element as they do in an fp32 product.
// Block = four wavefronts stacked in K over one 128-column strip; the grid is sized so that every block is resident
// at once (two blocks per CU: the accumulators of 64 rows x 128 columns take 128 registers).  Slab partials and the
// finishing launch are those of the form above.
constexpr int kMmaStripCols = 128; // 32 lane columns x float4
constexpr int kMmaTileRows = 16;   // k of the instruction
constexpr int kMmaWaves = 4;

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

struct MmaPlan {
  int64_t strips, tiles, tiles_per_wave, slabs;
};
__host__ __device__ inline MmaPlan mma_plan(int64_t K, int64_t N) {
  MmaPlan p;
  p.strips = ceil_div(N, kMmaStripCols);
  p.tiles = K / kMmaTileRows;
  int64_t want = 512 / p.strips; // blocks that are resident at once: 256 CUs x 2
  if (want < 1)
    want = 1;
  p.tiles_per_wave = ceil_div(p.tiles, want * kMmaWaves);
  p.slabs = ceil_div(p.tiles, p.tiles_per_wave * kMmaWaves);
  return p;
}

// Upper halves of two words: (hi & 0xffff0000) | (lo >> 16).
__device__ __forceinline__ uint32_t upper_halves(uint32_t hi, uint32_t lo) {
  return __builtin_amdgcn_perm(hi, lo, 0x07060302u);
}

// Byte pointers into global memory that every lane holds the same value of, moved to scalar registers: the loads
// and stores then take the scalar base + 32-bit lane offset form, and no lane computes 64-bit addresses.
typedef __attribute__((address_space(1))) char global_char_t;
__device__ __forceinline__ global_char_t *uniform_global(const void *p, uint64_t byte_offset) {
  const uint64_t v = reinterpret_cast<uint64_t>(p) + byte_offset;
  const uint64_t u = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
  return reinterpret_cast<global_char_t *>(u);
}

template <int kMF, bool kFull>
__device__ __forceinline__ void few_rows_mma_walk(const float *__restrict__ W, float *__restrict__ Wb,
                                                  const float *__restrict__ x, int64_t M, int64_t K, int64_t N,
                                                  int t0, int t1, int64_t n0, float zero_to,
                                                  f32x16_t (&acc)[kMF][4], float (&cs)[4]) {
  const int lane = threadIdx.x & 63;
  const int h = lane >> 5, c = lane & 31;
  const bool col_ok = kFull || n0 < N;
  const int64_t n_ld = col_ok ? n0 : N - 4; // loads are unconditional: a clamped address, masked afterwards
  const uint32_t lane_bytes = (uint32_t)((8 * h * N + n_ld) * 4);
  const uint64_t row_bytes = (uint64_t)N * 4, tile_bytes = row_bytes * kMmaTileRows;
  // this lane's rows of x (clamped; rows past M are zeroed after the load) at k = 8h .. 8h+7 of a tile
  uint32_t x_lane_bytes[kMF];
  bool row_ok[kMF];
#pragma unroll
  for (int f = 0; f < kMF; ++f) {
    const int64_t m = 32 * f + c;
    row_ok[f] = kFull || m < M;
    x_lane_bytes[f] = (uint32_t)(((row_ok[f] ? m : M - 1) * K + 8 * h) * 4);
  }
  // running positions (uniform): the next tile to load, the tile whose signs are stored next
  const global_char_t *w_next = uniform_global(W, (uint64_t)t0 * tile_bytes);
  const global_char_t *x_next = uniform_global(x, (uint64_t)t0 * (kMmaTileRows * 4));
  global_char_t *wb_next = uniform_global(Wb, (uint64_t)t0 * tile_bytes);
  typedef const __attribute__((address_space(1))) float4_t global_f4_t;
  struct Tile {
    float4_t w[8];
    float4_t x[kMF][2];
  };
  // (`more` false: the last tile again, so that the loop body has no branch; nothing uses what arrives)
  auto load_tile = [&](Tile &d, bool more) {
    const global_char_t *ws = more ? w_next : w_next - tile_bytes, *xs = more ? x_next : x_next - kMmaTileRows * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      d.w[j] = *reinterpret_cast<global_f4_t *>(ws + j * row_bytes + lane_bytes);
#pragma unroll
    for (int f = 0; f < kMF; ++f) {
      d.x[f][0] = *reinterpret_cast<global_f4_t *>(xs + x_lane_bytes[f]);
      d.x[f][1] = *reinterpret_cast<global_f4_t *>(xs + x_lane_bytes[f] + 16);
    }
    w_next += tile_bytes;
    x_next += kMmaTileRows * 4;
  };
  // One tile is in registers at a time: its successor is requested as soon as the operands have been formed from it
  // (the registers of the raw weights are free then) and arrives while the products run and the other wavefronts
  // of the CU work on theirs.
  auto consume_tile = [&](Tile &d, bool more) {
    // A: three bf16 terms of eight x values per row fragment
    u32x4_t a_hi[kMF], a_mid[kMF], a_lo[kMF];
#pragma unroll
    for (int f = 0; f < kMF; ++f) {
      uint32_t th[8], tm[8], tl[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float v = d.x[f][j >> 2][j & 3];
        if (!kFull && !row_ok[f])
          v = 0.0f;
        const uint32_t b = __float_as_uint(v);
        const bool finite = (b & 0x7f800000u) != 0x7f800000u;
        // a NaN whose payload sits in the lower half must not be cut down to an infinity
        const uint32_t top = (finite || (b & 0x007fffffu) == 0u) ? (b & 0xffff0000u) : 0x7fc00000u;
        const float r1 = finite ? v - __uint_as_float(top) : 0.0f; // exact
        const uint32_t mid = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(mid);                // exact, at most eight significant bits
        th[j] = top, tm[j] = mid, tl[j] = __float_as_uint(r2);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a_hi[f][i] = upper_halves(th[2 * i + 1], th[2 * i]);
        a_mid[f][i] = upper_halves(tm[2 * i + 1], tm[2 * i]);
        a_lo[f][i] = upper_halves(tl[2 * i + 1], tl[2 * i]);
      }
    }
    // B: signs of the tile, also the function's output Wb; |W| column sums
    u32x4_t b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4_t s[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float4_t w = d.w[2 * i + e];
        s[e].x = sign_of(w.x, zero_to), s[e].y = sign_of(w.y, zero_to);
        s[e].z = sign_of(w.z, zero_to), s[e].w = sign_of(w.w, zero_to);
        if (col_ok)
          __builtin_nontemporal_store(s[e], reinterpret_cast<__attribute__((address_space(1))) float4_t *>(
                                                wb_next + (2 * i + e) * row_bytes + lane_bytes));
        cs[0] += fabsf(w.x), cs[1] += fabsf(w.y), cs[2] += fabsf(w.z), cs[3] += fabsf(w.w);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q)
        b[q][i] = upper_halves(__float_as_uint(s[1][q]), __float_as_uint(s[0][q]));
    }
    wb_next += tile_bytes;
    __builtin_amdgcn_sched_barrier(0);
    load_tile(d, more);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bf16x8_t vb = __builtin_bit_cast(bf16x8_t, b[q]);
#pragma unroll
      for (int f = 0; f < kMF; ++f) { // smallest terms first
        acc[f][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_lo[f]), vb, acc[f][q], 0, 0, 0);
        acc[f][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_mid[f]), vb, acc[f][q], 0, 0, 0);
        acc[f][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_hi[f]), vb, acc[f][q], 0, 0, 0);
      }
    }
  };
  if (t0 >= t1)
    return;
  Tile tile;
  load_tile(tile, true);
#pragma clang loop unroll(disable)
  for (int t = t0; t < t1; ++t)
    consume_tile(tile, t + 1 < t1);
}

// partial[slab][r][Npad]: r < 32 kMF the dot products of input row r over the slab, r == 32 kMF the |W| column sums.
template <int kMF>
__global__ __launch_bounds__(64 * kMmaWaves, 2) void binary_affine_few_rows_mma(
    const float *__restrict__ W, float *__restrict__ Wb, const float *__restrict__ x, float *__restrict__ partial,
    int64_t M, int64_t K, int64_t N, int64_t Npad, int64_t tiles_per_wave, float zero_to) {
  constexpr int MT = 32 * kMF;
  constexpr int kVals = 4 * 16 + 4; // one row fragment's accumulators per lane, and the column sums
  __shared__ __attribute__((aligned(16))) float red[2 * kVals * 64];

  const int lane = threadIdx.x & 63;
  const int wk = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = lane >> 5, c = lane & 31;
  const int64_t slab = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * kMmaStripCols + 4 * c;
  // this wavefront's tiles (uniform, kept in scalar registers)
  const int tiles = (int)(K / kMmaTileRows), per = (int)tiles_per_wave;
  int t0 = __builtin_amdgcn_readfirstlane(((int)slab * kMmaWaves + wk) * per), t1 = t0 + per;
  t0 = t0 < tiles ? t0 : tiles;
  t1 = t1 < tiles ? t1 : tiles;

  f32x16_t acc[kMF][4];
  float cs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int f = 0; f < kMF; ++f)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[f][q][r] = 0.0f;

  const bool full = ((int64_t)blockIdx.x + 1) * kMmaStripCols <= N && M == MT;
  if (full)
    few_rows_mma_walk<kMF, true>(W, Wb, x, M, K, N, t0, t1, n0, zero_to, acc, cs);
  else
    few_rows_mma_walk<kMF, false>(W, Wb, x, M, K, N, t0, t1, n0, zero_to, acc, cs);

  // the two halves of a wavefront walked different rows of the same columns
#pragma unroll
  for (int q = 0; q < 4; ++q)
    cs[q] += __shfl_xor(cs[q], 32);

  // Fold over wk in a fixed order, (wk0 + wk2) + (wk1 + wk3), through LDS, one row fragment at a time.
  auto slot = [&](int s) { return red + (size_t)s * kVals * 64 + lane; };
#pragma unroll
  for (int f = 0; f < kMF; ++f) {
    auto put = [&](float *dst) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          dst[(q * 16 + r) * 64] = acc[f][q][r];
      if (f == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          dst[(64 + q) * 64] = cs[q];
      }
    };
    auto add = [&](const float *src) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[f][q][r] += src[(q * 16 + r) * 64];
      if (f == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          cs[q] += src[(64 + q) * 64];
      }
    };
    if (f > 0)
      __syncthreads();
    if (wk >= 2)
      put(slot(wk - 2));
    __syncthreads();
    if (wk < 2)
      add(slot(wk));
    __syncthreads();
    if (wk == 1)
      put(slot(1));
    __syncthreads();
    if (wk == 0)
      add(slot(1));
  }
  if (wk != 0)
    return;
  // accumulator register r of lane (h, c): input row 8 (r / 4) + 4 h + r % 4 of the fragment, columns 4c .. 4c+3
  float *out = partial + (size_t)slab * (MT + 1) * Npad + n0; // n0 < Npad always
#pragma unroll
  for (int f = 0; f < kMF; ++f)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = 32 * f + 8 * (r >> 2) + 4 * h + (r & 3);
      if (m < M) {
        float4_t o;
        o.x = acc[f][0][r], o.y = acc[f][1][r], o.z = acc[f][2][r], o.w = acc[f][3][r];
        *reinterpret_cast<float4_t *>(out + (size_t)m * Npad) = o;
      }
    }
  if (h == 0) {
    float4_t o;
    o.x = cs[0], o.y = cs[1], o.z = cs[2], o.w = cs[3];
    *reinterpret_cast<float4_t *>(out + (size_t)MT * Npad) = o;
  }
}

template <int kMF>
int launch_few_rows_mma(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                        int64_t M, int64_t K, int64_t N, float zero_to, float *partial, hipStream_t stream) {
  constexpr int MT = 32 * kMF;
  const MmaPlan p = mma_plan(K, N);
  const int64_t Npad = small_m_padded_cols(N);
  hipLaunchKernelGGL((binary_affine_few_rows_mma<kMF>), dim3((unsigned)p.strips, (unsigned)p.slabs),
                     dim3(64 * kMmaWaves), 0, stream, W, Wb, x, partial, M, K, N, Npad, p.tiles_per_wave, zero_to);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_few_rows_mma");
  hipLaunchKernelGGL(binary_affine_small_m_finish<MT>, dim3((unsigned)ceil_div(N / 4, 256), (unsigned)M), dim3(256), 0,
                     stream, partial, alpha, bias, y, M, N, Npad, p.slabs, (float)1 / K);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_small_m_finish");
  return NBLA_HIP_OK;
}

} // namespace

// From kMmaFromRows rows on the matrix-core walk is the faster one; it needs whole 16-row tiles of W and 16-byte
// loads of x.  Up to kSmallMMaxRows rows the vector-ALU walk takes what it does not cover.
constexpr int64_t kMmaFromRows = 9;
static bool few_rows_mma_applies(const float *x, int64_t M, int64_t K, int64_t N, float zero_to) {
  // (lane offsets into x and W are 32-bit byte counts; the sign operand is the upper half of the fp32 sign, so
  // Sign(0) = zero_to must be a value bf16 holds exactly)
  uint32_t zero_to_bits;
  memcpy(&zero_to_bits, &zero_to, sizeof zero_to_bits);
  return M >= kMmaFromRows && M <= kFewRowsMaxRows && K >= kMmaTileRows && K % kMmaTileRows == 0 &&
         K < (1ll << 23) && aligned16(x) && N < (1ll << 26) && (zero_to_bits & 0xffffu) == 0 &&
         mma_plan(K, N).slabs <= 65535;
}

bool small_m_affine_applies(const float *x, const float *W, const float *Wb, const float *alpha, const float *bias,
                            const float *y, int64_t M, int64_t K, int64_t N, float zero_to) {
  // (the vector-ALU walk addresses a row of W with 32-bit byte offsets)
  if (!(M >= 1 && K >= 1 && N % 4 == 0 && N < (1ll << 29) && Wb && aligned16(W) && aligned16(Wb) && aligned16(y) &&
        aligned16(alpha) && aligned16(bias)))
    return false;
  return few_rows_mma_applies(x, M, K, N, zero_to) || (M <= kSmallMMaxRows && small_m_slabs(K) <= 65535);
}

// (sized without knowing x: the larger of the two forms where both may run)
size_t small_m_affine_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M < 1 || M > kFewRowsMaxRows)
    return 0;
  size_t bytes = 0;
  if (M >= kMmaFromRows && K % kMmaTileRows == 0) {
    const int64_t mt = M <= 32 ? 32 : 64;
    bytes = (size_t)mma_plan(K, N).slabs * (mt + 1) * small_m_padded_cols(N) * sizeof(float);
  }
  if (M <= kSmallMMaxRows) {
    const int64_t mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const size_t valu = (size_t)small_m_slabs(K) * (mt + 1) * small_m_padded_cols(N) * sizeof(float);
    bytes = valu > bytes ? valu : bytes;
  }
  return bytes;
}

int launch_small_m_affine(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                          int64_t M, int64_t K, int64_t N, float zero_to, void *workspace, size_t workspace_bytes,
                          hipStream_t stream) {
  if (workspace_bytes < small_m_affine_workspace_bytes(M, K, N) || !aligned16(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "small-M binary affine workspace too small or misaligned.");
  float *partial = static_cast<float *>(workspace);
  if (few_rows_mma_applies(x, M, K, N, zero_to)) {
    if (M <= 32)
      return launch_few_rows_mma<1>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
    return launch_few_rows_mma<2>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
  }
  if (M > kSmallMMaxRows)
    return fail(NBLA_HIP_ERR_VALUE, "small-M binary affine: shape not covered (M=%lld, K=%lld).", (long long)M,
                (long long)K);
  if (M <= 1)
    return launch_small_m<1, 4>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
  if (M <= 2)
    return launch_small_m<2, 4>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
  if (M <= 4)
    return launch_small_m<4, 4>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
  if (M <= 8)
    return launch_small_m<8, 4>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
  return launch_small_m<16, 4>(x, W, Wb, alpha, bias, y, M, K, N, zero_to, partial, stream);
}

} // namespace nbla_hip
