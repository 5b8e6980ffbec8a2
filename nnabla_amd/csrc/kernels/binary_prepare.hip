// Operand preparation for the binary-weight products: one pass over W that
// writes Sign(W), the 1-bit packed MFMA operand and the |W| column sums, and the
// int8 digit operands of the activations.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

#include <cmath>

namespace nbla_hip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kPrepBlock = 256;
constexpr int kKSlice = 512; // k rows handled by one block of binarize_kn (16 k-tiles)

// sign.hpp:48-50
__device__ __forceinline__ float sign_of(float w, float zero_to) {
  return (w > 0.0f) ? 1.0f : ((w < 0.0f) ? -1.0f : zero_to);
}

// Workspace: colsum partials [slices][Np] floats, then zero-count partials
// [slices * col_groups] ints, then the pair words.  slices depends on the source layout.
struct PrepPlan {
  int64_t k_tiles, col_groups, Np, slices;
  int64_t wide_groups, Npw, slabs; // the streaming [K, N] kernel: 256-column groups, padded columns, slabs of 256 rows
  size_t sums_bytes, zeros_bytes, pairs_bytes;
};

PrepPlan make_prep_plan(int64_t K, int64_t N, bool transposed) {
  PrepPlan P;
  P.k_tiles = bits_k_tiles(K);
  P.col_groups = bits_col_groups(N);
  P.Np = P.col_groups * kColGroup;
  // the scalar [K, N] kernel covers 16 k tiles per block, the [N, K] kernels 4; size for the finer one
  P.slices = transposed ? ceil_div(P.k_tiles, 4) : ceil_div(P.k_tiles, 8);
  P.wide_groups = bits_wide_groups(N);
  P.Npw = P.wide_groups * kWideGroup;
  P.slabs = bits_packed_k_tiles(K) / 8;
  // (matrices of few blocks use slabs of 128 rows: twice the partial sums)
  const size_t sums_a = (size_t)P.slices * P.Np, sums_b = transposed ? 0 : (size_t)2 * P.slabs * P.Npw;
  P.sums_bytes = round_up((sums_a > sums_b ? sums_a : sums_b) * sizeof(float), 256);
  P.zeros_bytes = round_up((size_t)P.slices * P.col_groups * sizeof(int), 256);
  P.pairs_bytes = round_up((size_t)P.k_tiles * P.col_groups * 64 * sizeof(uint32_t), 256);
  return P;
}

// W stored [K, N].  Block = 16 teams of 16 threads; team t handles k-tile
// (slice * 16 + t) of column group blockIdx.x.  Thread (nq, g) of a team owns
// columns f*32 + 4*nq + {0..3} (f = 0, 1) and k offsets g*16 + {0..15}:
// 32 bits for each of four packed words, which are exactly the words of lanes
// g*32 + 4*nq + {0..3}.
template <bool kVec>
__global__ __launch_bounds__(kPrepBlock) void binarize_kn(const float *__restrict__ W, float *__restrict__ Wb,
                                                          uint32_t *__restrict__ bits, float *__restrict__ sums,
                                                          int *__restrict__ zeros, int64_t K, int64_t N,
                                                          int64_t col_groups, int64_t Np, float zero_to) {
  const int team = threadIdx.x >> 4, tt = threadIdx.x & 15;
  const int nq = tt & 7, g = tt >> 3;
  const int64_t cg = blockIdx.x;
  const int64_t kt = (int64_t)blockIdx.y * 16 + team;
  uint32_t word[4] = {0u, 0u, 0u, 0u};
  float asum[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  int nzero = 0;
  if (kt * kTileK < K) {
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      const int64_t n0 = cg * kColGroup + f * 32 + 4 * nq;
      {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int64_t k = kt * kTileK + g * 16 + j;
          if (k >= K || n0 >= N)
            continue;
          float w[4];
          if (kVec) {
            const float4_t v = *reinterpret_cast<const float4_t *>(W + k * N + n0);
            w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
          } else {
#pragma unroll
            for (int c = 0; c < 4; ++c)
              w[c] = (n0 + c < N) ? W[k * N + n0 + c] : 1.0f;
          }
          float b[4];
          const int pos = packed_bit_position(f, j);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            b[c] = sign_of(w[c], zero_to);
            const bool in = kVec || (n0 + c < N);
            const bool is_zero = !(w[c] > 0.0f) && !(w[c] < 0.0f); // +-0 (and NaN) take zero_to
            const bool neg = (w[c] < 0.0f) || (is_zero && zero_to < 0.0f);
            word[c] |= (in && neg) ? (1u << pos) : 0u;
            asum[f][c] += in ? fabsf(w[c]) : 0.0f;
            nzero += (in && is_zero) ? 1 : 0;
          }
          if (!Wb) {
          } else if (kVec) {
            float4_t o;
            o.x = b[0], o.y = b[1], o.z = b[2], o.w = b[3];
            *reinterpret_cast<float4_t *>(Wb + k * N + n0) = o;
          } else {
#pragma unroll
            for (int c = 0; c < 4; ++c)
              if (n0 + c < N)
                Wb[k * N + n0 + c] = b[c];
          }
        }
      }
    }
    uint4_t wv;
    wv.x = word[0], wv.y = word[1], wv.z = word[2], wv.w = word[3];
    *reinterpret_cast<uint4_t *>(bits + (kt * col_groups + cg) * 64 + g * 32 + 4 * nq) = wv;
  }
  // |W| column sums of this k slice: fixed-order fold of the 32 (team, g) partials.
  __shared__ float s_sum[32][kColGroup];
  __shared__ int s_zero[kPrepBlock / 64];
#pragma unroll
  for (int f = 0; f < 2; ++f)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      s_sum[team * 2 + g][f * 32 + 4 * nq + c] = asum[f][c];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    nzero += __shfl_xor(nzero, off);
  if ((threadIdx.x & 63) == 0)
    s_zero[threadIdx.x >> 6] = nzero;
  __syncthreads();
  if (threadIdx.x < kColGroup) {
    float acc = 0.0f;
    for (int r = 0; r < 32; ++r)
      acc += s_sum[r][threadIdx.x];
    sums[(int64_t)blockIdx.y * Np + cg * kColGroup + threadIdx.x] = acc;
  }
  if (threadIdx.x == 0)
    zeros[(int64_t)blockIdx.y * col_groups + cg] = s_zero[0] + s_zero[1] + s_zero[2] + s_zero[3];
}

// W stored [K, N], N % 4 == 0, 16-byte aligned: the streaming path.  A block of four wavefronts covers 256 rows of one
// 256-column group, wavefront w rows 64 w .. 64 w + 63 (two k tiles); a lane owns four consecutive columns, so every
// load and store instruction of a wavefront moves 1 KiB of one row.  Four rows are in flight while four are consumed
// (128 registers per lane: sixteen wavefronts per CU).
// Per element: Sign -> Wb (nontemporal store), |w| into the lane's column sums, the sign bit shifted into a 32-bit
// word per column (bit k = row k of the k tile).  After 32 rows the wavefront transposes those words through LDS into
// the packed operand's own layout (lane l: columns F * 32 + l % 32, k slots (l / 32) * 16 + j; bit F + 8 c of word i
// for k slot 4 i + c) and writes the k tile's 1 KiB straight into the packed operand.  No intermediate pair words and
// no relayout pass.  Column sums: lanes in row order, then the block's four wavefronts through LDS in wavefront order.
constexpr int kWideBatch = 4;
constexpr int kWideTileBatches = kTileK / kWideBatch; // batches per k tile
// kAligned: N a multiple of four and 16-byte aligned W / Wb, a lane's four columns are one 128-bit access; otherwise
// four 32-bit ones, each column clamped and masked on its own (a row of W then starts at any multiple of four bytes).
template <int kWideWaveRows, bool kFull, bool kCountZeros, bool kAligned>
__device__ __forceinline__ void binarize_wide_walk(const float *__restrict__ W, float *__restrict__ Wb,
                                                   uint4_t *__restrict__ bits_out, int64_t tile_stride, uint32_t *s_x,
                                                   int64_t K, int64_t N, int64_t k_wave, int64_t n0, int lane,
                                                   float zero_to,
                                                   float (&cs)[4], int &nzero) {
  const bool col_ok = kFull || n0 < N;
  const int64_t n_ld = col_ok ? n0 : N - 4; // loads are unconditional: a clamped address, masked afterwards
  const uint32_t lane_bytes = (uint32_t)(n_ld * 4);
  uint32_t col_bytes[4];
  bool col_in[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    col_in[c] = kFull || n0 + c < N;
    col_bytes[c] = (uint32_t)((col_in[c] ? n0 + c : N - 1) * 4);
  }
  float4_t va[kWideBatch], vb[kWideBatch];
  uint32_t word[4] = {0u, 0u, 0u, 0u};
  auto load_batch = [&](int b, float4_t (&dst)[kWideBatch]) {
#pragma unroll
    for (int j = 0; j < kWideBatch; ++j) {
      int64_t k = k_wave + b * kWideBatch + j;
      if (!kFull && k >= K)
        k = K - 1;
      const char *row = reinterpret_cast<const char *>(W + k * N); // uniform base + 32-bit lane offset
      if (kAligned) {
        dst[j] = *reinterpret_cast<const float4_t *>(row + lane_bytes);
      } else {
        dst[j].x = *reinterpret_cast<const float *>(row + col_bytes[0]);
        dst[j].y = *reinterpret_cast<const float *>(row + col_bytes[1]);
        dst[j].z = *reinterpret_cast<const float *>(row + col_bytes[2]);
        dst[j].w = *reinterpret_cast<const float *>(row + col_bytes[3]);
      }
    }
  };
  auto consume_batch = [&](int b, const float4_t (&src)[kWideBatch]) {
#pragma unroll
    for (int j = 0; j < kWideBatch; ++j) {
      const int64_t k = k_wave + b * kWideBatch + j;
      const bool row_in = kFull || k < K;
      const float w[4] = {src[j].x, src[j].y, src[j].z, src[j].w};
      float sg[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bool in = kAligned ? (kFull || (col_ok && row_in)) : (row_in && col_in[c]);
        // sign.hpp:48-50; +-0 and NaN are exactly the inputs that are neither less nor greater than zero
        const bool nonzero = __builtin_islessgreater(w[c], 0.0f);
        const float one = __uint_as_float((__float_as_uint(w[c]) & 0x80000000u) | 0x3f800000u);
        sg[c] = nonzero ? one : zero_to;
        // the sign of Sign(w) is the packed bit: rows enter at bit 31 and move down one place per row
        const uint32_t bit = in ? (__float_as_uint(sg[c]) & 0x80000000u) : 0u;
        word[c] = (word[c] >> 1) | bit;
        cs[c] += in ? fabsf(w[c]) : 0.0f;
        if (kCountZeros)
          nzero += (in && !nonzero) ? 1 : 0;
      }
      if (Wb && kAligned && (kFull || (col_ok && row_in))) {
        float4_t o;
        o.x = sg[0], o.y = sg[1], o.z = sg[2], o.w = sg[3];
        char *row = reinterpret_cast<char *>(Wb + k * N);
        __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(row + lane_bytes));
      }
      if (Wb && !kAligned && row_in) {
        char *row = reinterpret_cast<char *>(Wb + k * N);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col_in[c])
            __builtin_nontemporal_store(sg[c], reinterpret_cast<float *>(row + col_bytes[c]));
      }
    }
  };
  // 32 rows are in `word`: transpose them into the packed layout and write the k tile
  auto emit_tile = [&](int t) {
    uint4_t mine;
    mine.x = word[0], mine.y = word[1], mine.z = word[2], mine.w = word[3];
    *reinterpret_cast<uint4_t *>(s_x + 4 * lane) = mine;
    __builtin_amdgcn_wave_barrier(); // the wavefront's own LDS traffic stays in program order
    const int q = (lane & 31) >> 2, c = lane & 3, half = (lane >> 5) * 16;
    uint32_t out[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int F = 0; F < 8; ++F) {
      const uint32_t col = s_x[(F * 8 + q) * 4 + c]; // column F * 32 + lane % 32, bit k = row k
      const uint32_t h = (col >> half) & 0xffffu;    // this lane's sixteen k slots
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t nib = (h >> (4 * i)) & 0xfu;
        // bits 0..3 of nib to bit positions 0, 8, 16, 24 (the sixteen partial products land on distinct bits)
        out[i] |= ((nib * 0x00204081u) & 0x01010101u) << F;
      }
    }
    __builtin_amdgcn_wave_barrier();
    uint4_t o;
    o.x = out[0], o.y = out[1], o.z = out[2], o.w = out[3];
    bits_out[(size_t)t * tile_stride] = o; // bits_out: this lane's slot in the wavefront's first k tile
  };
  constexpr int kBatches = kWideWaveRows / kWideBatch;
  load_batch(0, va);
#pragma clang loop unroll(disable)
  for (int b = 0; b < kBatches; b += 2) {
    load_batch(b + 1, vb);
    consume_batch(b, va);
    if (b + 2 < kBatches)
      load_batch(b + 2, va);
    consume_batch(b + 1, vb);
    if ((b + 2) % kWideTileBatches == 0) {
      emit_tile(b / kWideTileBatches);
#pragma unroll
      for (int c = 0; c < 4; ++c)
        word[c] = 0u;
    }
  }
}

// kWideWaveRows: 64 (two k tiles per wavefront), or 32 for matrices that would otherwise give the CUs too few blocks.
template <int kWideWaveRows, bool kCountZeros, bool kAligned>
__global__ __launch_bounds__(kPrepBlock, 4) void binarize_kn_wide(const float *__restrict__ W, float *__restrict__ Wb,
                                                                 uint4_t *__restrict__ bits, float *__restrict__ sums,
                                                                 int *__restrict__ zeros, int64_t K, int64_t N,
                                                                 int64_t wide_groups, int64_t Npw, float zero_to) {
  __shared__ __attribute__((aligned(16))) uint32_t s_x[kPrepBlock / 64][256];
  __shared__ float s_sum[kPrepBlock / 64][kWideGroup];
  __shared__ int s_zero[kPrepBlock / 64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform: row indices stay in scalar registers
  const int64_t wg = blockIdx.x, slab = blockIdx.y;
  const int64_t k_wave = (slab * (kPrepBlock / 64) + wave) * kWideWaveRows;
  const int64_t n0 = wg * kWideGroup + 4 * lane;
  float cs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int nzero = 0;
  // consecutive k tiles of one wide group lie wide_groups * 64 uint4 apart
  uint4_t *tile0 = bits + ((k_wave / kTileK) * wide_groups + wg) * 64 + lane;
  const int64_t tile_stride = wide_groups * 64;
  const bool full = k_wave + kWideWaveRows <= K && (wg + 1) * kWideGroup <= N;
  if (full)
    binarize_wide_walk<kWideWaveRows, true, kCountZeros, kAligned>(W, Wb, tile0, tile_stride, s_x[wave], K, N, k_wave, n0,
                                                                   lane, zero_to, cs, nzero);
  else
    binarize_wide_walk<kWideWaveRows, false, kCountZeros, kAligned>(W, Wb, tile0, tile_stride, s_x[wave], K, N, k_wave, n0,
                                                                    lane, zero_to, cs, nzero);
  // column sums of the block's 256 rows, wavefronts in order
  *reinterpret_cast<float4_t *>(&s_sum[wave][4 * lane]) = float4_t{cs[0], cs[1], cs[2], cs[3]};
  if (kCountZeros) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      nzero += __shfl_xor(nzero, off);
    if (lane == 0)
      s_zero[wave] = nzero;
  }
  __syncthreads();
  sums[slab * Npw + wg * kWideGroup + threadIdx.x] =
      ((s_sum[0][threadIdx.x] + s_sum[1][threadIdx.x]) + s_sum[2][threadIdx.x]) + s_sum[3][threadIdx.x];
  if (kCountZeros && threadIdx.x == 0)
    zeros[slab * wide_groups + wg] = s_zero[0] + s_zero[1] + s_zero[2] + s_zero[3];
}

// W stored [N, K] (convolution weights viewed [channels_o, col_w]).  Wavefront w
// of the block handles k-tile blockIdx.y*4 + w of column group blockIdx.x; lane
// l builds its own packed word from 16 consecutive k of each of its two rows n(f).
__global__ __launch_bounds__(kPrepBlock) void binarize_nk(const float *__restrict__ W, float *__restrict__ Wb,
                                                          uint32_t *__restrict__ bits, float *__restrict__ sums,
                                                          int *__restrict__ zeros, int64_t K, int64_t N,
                                                          int64_t col_groups, int64_t Np, int64_t k_tiles,
                                                          float zero_to) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 5, r = lane & 31;
  const int64_t cg = blockIdx.x;
  const int64_t kt = (int64_t)blockIdx.y * 4 + wave;
  uint32_t word = 0u;
  float asum[2] = {0.f, 0.f};
  int nzero = 0;
  if (kt < k_tiles) {
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      const int64_t n = cg * kColGroup + f * 32 + r;
      {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int64_t k = kt * kTileK + g * 16 + j;
          if (n < N && k < K) {
            const float w = W[n * K + k];
            if (Wb)
              Wb[n * K + k] = sign_of(w, zero_to);
            const bool is_zero = !(w > 0.0f) && !(w < 0.0f);
            const bool neg = (w < 0.0f) || (is_zero && zero_to < 0.0f);
            word |= neg ? (1u << packed_bit_position(f, j)) : 0u;
            asum[f] += fabsf(w);
            nzero += is_zero ? 1 : 0;
          }
        }
      }
    }
    bits[(kt * col_groups + cg) * 64 + lane] = word;
  }
  __shared__ float s_sum[8][kColGroup];
  __shared__ int s_zero[kPrepBlock / 64];
  s_sum[wave * 2 + g][r] = asum[0];
  s_sum[wave * 2 + g][32 + r] = asum[1];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    nzero += __shfl_xor(nzero, off);
  if (lane == 0)
    s_zero[wave] = nzero;
  __syncthreads();
  if (threadIdx.x < kColGroup) {
    float acc = 0.0f;
    for (int q = 0; q < 8; ++q)
      acc += s_sum[q][threadIdx.x];
    sums[(int64_t)blockIdx.y * Np + cg * kColGroup + threadIdx.x] = acc;
  }
  if (threadIdx.x == 0)
    zeros[(int64_t)blockIdx.y * col_groups + cg] = s_zero[0] + s_zero[1] + s_zero[2] + s_zero[3];
}

// W stored [N, K], K % 4 == 0, 16-byte aligned: the streaming path of the layout above.  The block covers 64 rows
// x 128 k (slice blockIdx.x of column group blockIdx.y); thread t reads four consecutive k (one 128-bit load, 32
// lanes cover 512 contiguous bytes of a row) of rows i*8 + t/32, turns them into the four bits they occupy in the
// packed word (bit 4f + jq + 8c for k quad jq, element c) and parks that partial word in LDS; wavefront w then ORs
// the eight partial words (f, jq) of each packed word of k tile w.  |W| row sums: the four k of a thread in order,
// then a butterfly over the 32 lanes of the row.
constexpr int kPartStride = 36; // words per LDS row: 32 k quads + padding that keeps 16-byte alignment
template <bool kAligned> // false: rows of a length that is no multiple of four (or not 16-byte aligned), 32-bit accesses
__global__ __launch_bounds__(kPrepBlock) void binarize_nk_vec(const float *__restrict__ W, float *__restrict__ Wb,
                                                              uint32_t *__restrict__ bits, float *__restrict__ sums,
                                                              int *__restrict__ zeros, int64_t K, int64_t N,
                                                              int64_t col_groups, int64_t Np, int64_t k_tiles,
                                                              float zero_to) {
  __shared__ __attribute__((aligned(16))) uint32_t s_part[kColGroup * kPartStride];
  __shared__ int s_zero[kPrepBlock / 64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kq = threadIdx.x & 31, rsub = threadIdx.x >> 5;
  const int64_t slice = blockIdx.x, cg = blockIdx.y;
  const int64_t k = slice * 128 + kq * 4;
  float4_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t n = cg * kColGroup + i * 8 + rsub;
    if (kAligned) {
      if (n < N && k < K)
        v[i] = *reinterpret_cast<const float4_t *>(W + n * K + k);
      else
        v[i] = float4_t{1.0f, 1.0f, 1.0f, 1.0f};
    } else {
      const float *src = W + n * K + k;
      v[i].x = (n < N && k + 0 < K) ? src[0] : 1.0f;
      v[i].y = (n < N && k + 1 < K) ? src[1] : 1.0f;
      v[i].z = (n < N && k + 2 < K) ? src[2] : 1.0f;
      v[i].w = (n < N && k + 3 < K) ? src[3] : 1.0f;
    }
  }
  int nzero = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = i * 8 + rsub;
    const int64_t n = cg * kColGroup + row;
    const bool row_in = n < N && k < K;
    const float w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    float b[4];
    uint32_t part = 0u;
    float asum = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const bool in = kAligned ? row_in : (n < N && k + c < K);
      b[c] = sign_of(w[c], zero_to);
      const bool is_zero = !(w[c] > 0.0f) && !(w[c] < 0.0f);
      const bool neg = (w[c] < 0.0f) || (is_zero && zero_to < 0.0f);
      part |= (in && neg) ? (1u << (4 * (i >> 2) + (kq & 3) + 8 * c)) : 0u;
      asum += in ? fabsf(w[c]) : 0.0f;
      nzero += (in && is_zero) ? 1 : 0;
    }
    s_part[row * kPartStride + kq] = part;
    if (kAligned && row_in && Wb) {
      float4_t o;
      o.x = b[0], o.y = b[1], o.z = b[2], o.w = b[3];
      __builtin_nontemporal_store(o, reinterpret_cast<float4_t *>(Wb + n * K + k));
    }
    if (!kAligned && Wb) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (n < N && k + c < K)
          __builtin_nontemporal_store(b[c], Wb + n * K + k + c);
    }
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1)
      asum += __shfl_xor(asum, off);
    if (kq == 0)
      sums[slice * Np + cg * kColGroup + row] = asum;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    nzero += __shfl_xor(nzero, off);
  if (lane == 0)
    s_zero[wave] = nzero;
  __syncthreads();
  const int64_t kt = slice * 4 + wave;
  if (kt < k_tiles) {
    const int g = lane >> 5, r = lane & 31;
    uint32_t word = 0u;
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      const uint4_t q = *reinterpret_cast<const uint4_t *>(&s_part[(f * 32 + r) * kPartStride + wave * 8 + g * 4]);
      word |= q.x | q.y | q.z | q.w;
    }
    bits[(kt * col_groups + cg) * 64 + lane] = word;
  }
  if (threadIdx.x == 0)
    zeros[slice * col_groups + cg] = s_zero[0] + s_zero[1] + s_zero[2] + s_zero[3];
}

// Pair words -> packed operand: thread (k tile, wide group, lane) interleaves the four pair groups of its wide group.
__device__ __forceinline__ void widen_bits(const uint32_t *__restrict__ pairs, uint4_t *__restrict__ bits,
                                           int64_t k_tiles, int64_t col_groups, int64_t wide_groups, int64_t idx) {
  const int lane = (int)(idx & 63);
  const int64_t t = idx >> 6;
  const int64_t kt = t / wide_groups, wg = t - kt * wide_groups;
  uint32_t w[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    w[q] = (kt < k_tiles && 4 * wg + q < col_groups) ? pairs[(kt * col_groups + 4 * wg + q) * 64 + lane] : 0u;
  uint32_t o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int f = 0; f < 2; ++f)
        o[i] |= ((w[q] >> (4 * f + i)) & 0x01010101u) << (2 * q + f);
  uint4_t v;
  v.x = o[0], v.y = o[1], v.z = o[2], v.w = o[3];
  bits[idx] = v;
}

// alpha[n] = (sum over slices) * ((float)1 / K)   (binary_weight_affine.cpp:68,
// binary_weight_convolution.cpp:66: a multiply by the rounded reciprocal), and
// the total zero count; the same launch turns the pair words into the packed operand (one thread per output uint4).
__global__ __launch_bounds__(kPrepBlock) void binarize_finalize(const float *__restrict__ sums, const int *__restrict__ zeros,
                                                                float *__restrict__ alpha, int *__restrict__ zero_count,
                                                                int64_t N, int64_t Np, int64_t slices,
                                                                int64_t zero_entries, float inv_k,
                                                                const uint32_t *__restrict__ pairs,
                                                                uint4_t *__restrict__ bits, int64_t k_tiles,
                                                                int64_t col_groups, int64_t wide_groups,
                                                                int64_t widen_total) {
  const int64_t n = (int64_t)blockIdx.x * kPrepBlock + threadIdx.x;
  if (n < widen_total)
    widen_bits(pairs, bits, k_tiles, col_groups, wide_groups, n);
  if (alpha && n < N) {
    float acc = 0.0f;
    // eight slices' loads are issued before the first is added (the adds keep slice order)
    for (int64_t s0 = 0; s0 < slices; s0 += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        v[j] = sums[((s0 + j < slices) ? s0 + j : slices - 1) * Np + n];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < slices)
          acc += v[j];
    }
    alpha[n] = acc * inv_k;
  }
  if (zero_count && blockIdx.x == 0) {
    int z = 0;
    for (int64_t i = threadIdx.x; i < zero_entries; i += kPrepBlock)
      z += zeros[i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      z += __shfl_xor(z, off);
    __shared__ int s_z[kPrepBlock / 64];
    if ((threadIdx.x & 63) == 0)
      s_z[threadIdx.x >> 6] = z;
    __syncthreads();
    if (threadIdx.x == 0)
      *zero_count = s_z[0] + s_z[1] + s_z[2] + s_z[3];
  }
}

// ------------------------------------------------------------ digit operand
// Largest shift s with rint(amax * 2^s) <= kDigitMax, for amax > 0 finite given as its bit pattern.
__device__ __forceinline__ int digit_shift(uint32_t amax_bits) {
  const int e = binade_exponent(binade_of(amax_bits)); // amax in [2^e, 2^(e+1))
  int s = 22 - e;                                      // amax * 2^s in [2^22, 2^23)
  if (rintf(ldexpf(__uint_as_float(amax_bits), s)) > (float)kDigitMax)
    --s;
  return s;
}
__device__ __forceinline__ int to_fixed(float v, int s) { return (int)rintf(ldexpf(v, s)); }

// Sixteen fixed-point values of one lane -> its 16 bytes of each digit fragment.
__device__ __forceinline__ void store_digits(const int (&q)[16], uint4_t *dst, bool streaming) {
  uint32_t w[3][4];
  pack_digits(q, w);
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    uint4_t o;
    o.x = w[d][0], o.y = w[d][1], o.z = w[d][2], o.w = w[d][3];
    if (streaming)
      __builtin_nontemporal_store(o, dst + d * 64);
    else
      dst[d * 64] = o;
  }
}

// One wavefront per (padded) row: the row's shift and, per chunk of kChunkK columns, the sum of its fixed-point
// values.  The second sweep over the row is served by the caches.
// `cs` (may be null) scales column k of x by cs[k] before anything else: one rounded fp32 product per element.
__device__ __forceinline__ float4_t scaled4(float4_t v, const float *__restrict__ cs, int64_t k) {
  if (cs) {
    const float4_t c = *reinterpret_cast<const float4_t *>(cs + k);
    v.x = v.x * c.x, v.y = v.y * c.y, v.z = v.z * c.z, v.w = v.w * c.w;
  }
  return v;
}

template <bool kVec>
__global__ __launch_bounds__(kPrepBlock) void digit_row_scale(const float *__restrict__ x, int64_t ldx,
                                                              const float *__restrict__ cs,
                                                              long long *__restrict__ sums,
                                                              int32_t *__restrict__ shift, int64_t M, int64_t K,
                                                              int64_t rows, int64_t chunks) {
  const int lane = threadIdx.x & 63;
  const int64_t m = (int64_t)blockIdx.x * (kPrepBlock / 64) + (threadIdx.x >> 6);
  if (m >= rows)
    return;
  if (m == 0 && lane == 0)
    shift[rows] = 1; // the operand's flag word (behind the shifts): a row-scaled operand is never in the narrow form
  if (m >= M) {
    if (lane == 0)
      shift[m] = 0;
    for (int64_t c = lane; c < chunks; c += 64)
      sums[c * rows + m] = 0;
    return;
  }
  const float *row = x + m * ldx;
  uint32_t amax = 0u;
  // rows of up to 4096 values stay in registers between the two sweeps (16 float4 per lane)
  constexpr int kKeep = 16;
  const bool keep = kVec && K <= 256 * kKeep;
  float4_t kept[kKeep];
  if (keep) {
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const int64_t k = 4 * lane + 256 * i;
      kept[i] = (k < K) ? scaled4(*reinterpret_cast<const float4_t *>(row + k), cs, k) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const uint32_t a = __float_as_uint(kept[i].x) & 0x7fffffffu, b = __float_as_uint(kept[i].y) & 0x7fffffffu;
      const uint32_t c = __float_as_uint(kept[i].z) & 0x7fffffffu, d = __float_as_uint(kept[i].w) & 0x7fffffffu;
      amax = max(max(amax, max(a, b)), max(c, d));
    }
  } else if (kVec) {
    for (int64_t k = 4 * lane; k < K; k += 256) { // K % 4 == 0
      const float4_t v = scaled4(*reinterpret_cast<const float4_t *>(row + k), cs, k);
      const uint32_t a = __float_as_uint(v.x) & 0x7fffffffu, b = __float_as_uint(v.y) & 0x7fffffffu;
      const uint32_t c = __float_as_uint(v.z) & 0x7fffffffu, d = __float_as_uint(v.w) & 0x7fffffffu;
      amax = max(max(amax, max(a, b)), max(c, d));
    }
  } else {
    for (int64_t k = lane; k < K; k += 64)
      amax = max(amax, __float_as_uint(cs ? row[k] * cs[k] : row[k]) & 0x7fffffffu);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    amax = max(amax, (uint32_t)__shfl_xor((int)amax, off));
  const bool bad = amax >= 0x7f800000u;
  const int s = (bad || amax == 0u) ? 0 : digit_shift(amax);
  if (lane == 0)
    shift[m] = bad ? kBadRow : s;
  for (int64_t c = 0; c < chunks; ++c) {
    const int64_t k_begin = c * kChunkK, k_end = (k_begin + kChunkK < K) ? k_begin + kChunkK : K;
    long long acc = 0;
    if (!bad) {
      if (keep) { // a single chunk
        int part = 0; // at most 64 values of magnitude < 2^23 per lane
#pragma unroll
        for (int i = 0; i < kKeep; ++i)
          part += to_fixed(kept[i].x, s) + to_fixed(kept[i].y, s) + to_fixed(kept[i].z, s) + to_fixed(kept[i].w, s);
        acc = part;
      } else if (kVec) {
        for (int64_t k = k_begin + 4 * lane; k < k_end; k += 256) {
          const float4_t v = scaled4(*reinterpret_cast<const float4_t *>(row + k), cs, k);
          acc += (long long)to_fixed(v.x, s) + to_fixed(v.y, s) + to_fixed(v.z, s) + to_fixed(v.w, s);
        }
      } else {
        for (int64_t k = k_begin + lane; k < k_end; k += 64)
          acc += to_fixed(cs ? row[k] * cs[k] : row[k], s);
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      acc += __shfl_xor(acc, off);
    if (lane == 0)
      sums[c * rows + m] = acc;
  }
}

// One wavefront per (row block, k tile) fragment triple; lane l converts x[rb*32 + l%32][kt*32 + (l/32)*16 + 0..15].
__global__ __launch_bounds__(kPrepBlock) void split_digits(const float *__restrict__ x, int64_t ldx,
                                                           const float *__restrict__ cs,
                                                           const int32_t *__restrict__ shift, uint4_t *__restrict__ out,
                                                           int64_t M, int64_t K, int64_t k_tiles, int64_t frags) {
  const int64_t frag = (int64_t)blockIdx.x * (kPrepBlock / 64) + (threadIdx.x >> 6);
  if (frag >= frags)
    return;
  const int lane = threadIdx.x & 63;
  const int64_t rb = frag / k_tiles, kt = frag - rb * k_tiles;
  const int64_t m = rb * kFragRows + (lane & 31);
  const int64_t k0 = kt * kTileK + (lane >> 5) * 16;
  const int s = shift[m];
  int q[16];
#pragma unroll
  for (int j = 0; j < 16; ++j)
    q[j] = (m < M && k0 + j < K && s != kBadRow)
               ? to_fixed(cs ? x[m * ldx + k0 + j] * cs[k0 + j] : x[m * ldx + k0 + j], s)
               : 0;
  store_digits(q, out + frag * kDigits * 64 + lane, false);
}

// Streaming variant for K % 64 == 0, 16-byte aligned rows: a wavefront converts a 32-row x 64-k patch (two k tiles).
// Global loads are fully coalesced (16 lanes read 256 contiguous bytes of a row); the patch is turned into fragment
// order through a padded LDS tile.
__global__ __launch_bounds__(kPrepBlock) void split_digits_tiled(const float *__restrict__ x, int64_t ldx,
                                                                 const float *__restrict__ cs,
                                                                 const int32_t *__restrict__ shift,
                                                                 uint4_t *__restrict__ out, int64_t M, int64_t K,
                                                                 int64_t k_tiles, int64_t patches) {
  constexpr int kRowStride = 68; // floats: 64 + 4 padding keeps the 128-bit column reads conflict-free
  __shared__ float tile[kPrepBlock / 64][32 * kRowStride];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t patch = (int64_t)blockIdx.x * (kPrepBlock / 64) + wave;
  if (patch >= patches)
    return;
  const int64_t patches_per_row = k_tiles / 2;
  const int64_t rb = patch / patches_per_row, kq = patch - rb * patches_per_row;
  float *t = tile[wave];
  const int lr = lane >> 4, lc = (lane & 15) * 4;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = j * 4 + lr;
    const int64_t m = rb * kFragRows + row;
    float4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (m < M && kq * 64 + lc < K) // the k tiles are padded past K
      v = scaled4(*reinterpret_cast<const float4_t *>(x + m * ldx + kq * 64 + lc), cs, kq * 64 + lc);
    *reinterpret_cast<float4_t *>(t + row * kRowStride + lc) = v;
  }
  const int r = lane & 31, g = lane >> 5;
  const int s = shift[rb * kFragRows + r];
  // the tile is private to this wavefront: LDS operations of one wavefront complete in order
  __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    int q[16];
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const float4_t a = *reinterpret_cast<const float4_t *>(t + r * kRowStride + h * 32 + g * 16 + v4 * 4);
      const bool ok = s != kBadRow;
      q[v4 * 4 + 0] = ok ? to_fixed(a.x, s) : 0;
      q[v4 * 4 + 1] = ok ? to_fixed(a.y, s) : 0;
      q[v4 * 4 + 2] = ok ? to_fixed(a.z, s) : 0;
      q[v4 * 4 + 3] = ok ? to_fixed(a.w, s) : 0;
    }
    store_digits(q, out + ((rb * k_tiles + kq * 2 + h) * kDigits) * 64 + lane, true);
  }
}

// A row of x holding a NaN or an infinity cannot be scaled to integers: its shift becomes kBadRow and a matrix-core
// product can only leave NaN in its whole output row.  The reference's affine propagates such values element by
// element (affine.cpp:87-95: Inf * w = +-Inf, Inf - Inf = NaN, NaN anywhere = NaN), so a caller that has the
// materialised weights at hand lets the kernel that finds such a row -- rare -- compute its outputs right away, as
// plain fp32 dot products in the reference's order, and tells the product to leave the row alone.
__device__ __noinline__ void redo_marked_row(const float *__restrict__ xrow, const RowRedo &redo, int64_t m, int64_t K,
                                             int threads) {
  for (int64_t n = threadIdx.x; n < redo.N; n += threads) {
    const float a = redo.alpha ? redo.alpha[n] : 1.0f;
    float acc = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const float w = redo.alpha ? redo.Wb[k * redo.N + n] * a : redo.Wb[k * redo.N + n]; // the weight as multiplied
      acc = acc + xrow[k] * w;
    }
    redo.y[m * redo.N + n] = redo.bias ? acc + redo.bias[n] : acc;
  }
}

// Scale and digits in one pass for rows of up to 16384 values: a block of eight
// wavefronts keeps kRows rows in registers in fragment order.  Wavefront w owns the k tiles
// [w * kSlots * kPer, (w + 1) * kSlots * kPer), kSlots = 32 / kRows; lane r + kRows * (g + 2 * ts) holds, for row r,
// the 16 values of fragment half g of the tiles kSlots * t + ts, t < kPer.  Row maxima and row sums cross the
// wavefronts through LDS; every store instruction then writes runs of kRows * 16 bytes of a fragment (the other rows
// of the row block come from neighbouring blocks).  x is read once.
// kAligned false: rows that do not start at multiples of 16 bytes or whose length is no multiple of four -- a lane's
// four consecutive values come as four 32-bit loads, each checked against the row's end.
constexpr int kFusedWaves = 8;
template <int kRows, int kPer, bool kAligned>
__global__ __launch_bounds__(kFusedWaves * 64) void split_digits_rows(const float *__restrict__ x, int64_t ldx,
                                                                       const float *__restrict__ cs,
                                                                       long long *__restrict__ sums,
                                                                       int32_t *__restrict__ shift,
                                                                       uint4_t *__restrict__ out, int64_t M, int64_t K,
                                                                       int64_t k_tiles, int64_t rows, RowRedo redo) {
  static_assert(kRows == 4 || kRows == 8 || kRows == 16, "rows per block");
  static_assert(kPer * 16 < 256, "a lane's partial sum of kPer * 16 values below 2^23 fits an int");
  constexpr int kSlots = 32 / kRows;
  __shared__ uint32_t s_max[kFusedWaves][kRows];
  __shared__ uint32_t s_low[kFusedWaves][kRows];
  __shared__ long long s_sum[kFusedWaves][kRows];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane % kRows, g = (lane / kRows) & 1, ts = lane / (2 * kRows);
  const int64_t m = (int64_t)blockIdx.x * kRows + r;
  if (blockIdx.x == 0 && threadIdx.x == 0)
    shift[rows] = 1; // the operand's flag word: a row-scaled operand is never in the column operands' narrow form
  const float *row = x + m * ldx;
  float4_t v[kPer][4];
  uint32_t amax = 0u;
#pragma unroll
  for (int t = 0; t < kPer; ++t) {
    const int64_t k0 = (((int64_t)wave * kPer + t) * kSlots + ts) * kTileK + g * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t k = k0 + 4 * i;
      if (kAligned) {
        v[t][i] = (m < M && k < K) ? scaled4(*reinterpret_cast<const float4_t *>(row + k), cs, k)
                                   : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      } else {
        float e[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const bool in = m < M && k + c < K;
          e[c] = in ? row[k + c] : 0.0f;
          if (cs) // one rounded product per element, as scaled4
            e[c] = e[c] * (in ? cs[k + c] : 0.0f);
        }
        v[t][i] = float4_t{e[0], e[1], e[2], e[3]};
      }
    }
  }
#pragma unroll
  for (int t = 0; t < kPer; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t a = __float_as_uint(v[t][i].x) & 0x7fffffffu, b = __float_as_uint(v[t][i].y) & 0x7fffffffu;
      const uint32_t c = __float_as_uint(v[t][i].z) & 0x7fffffffu, d = __float_as_uint(v[t][i].w) & 0x7fffffffu;
      amax = max(max(amax, max(a, b)), max(c, d));
    }
#pragma unroll
  for (int off = kRows; off < 64; off <<= 1)
    amax = max(amax, (uint32_t)__shfl_xor((int)amax, off));
  if (lane < kRows)
    s_max[wave][lane] = amax;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kFusedWaves; ++w)
    amax = max(amax, s_max[w][r]);
  const bool bad = amax >= 0x7f800000u;
  const int s = (bad || amax == 0u) ? 0 : digit_shift(amax);
  uint32_t low = 0u; // OR of the two lower digits of the row's values: zero for a one-digit row
  int part = 0;
#pragma unroll
  for (int t = 0; t < kPer; ++t) {
    int q[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q[4 * i + 0] = bad ? 0 : to_fixed(v[t][i].x, s);
      q[4 * i + 1] = bad ? 0 : to_fixed(v[t][i].y, s);
      q[4 * i + 2] = bad ? 0 : to_fixed(v[t][i].z, s);
      q[4 * i + 3] = bad ? 0 : to_fixed(v[t][i].w, s);
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      part += q[j];
      low |= (uint32_t)q[j] & 0xffffu; // q = d0 * 65536 + d1 * 256 + d2: d1 = d2 = 0 exactly when this is zero
    }
    const int64_t kt = ((int64_t)wave * kPer + t) * kSlots + ts;
    if (kt < k_tiles) {
      const int64_t rb = m / kFragRows;
      store_digits(q, out + ((rb * k_tiles + kt) * kDigits) * 64 + (int)(m % kFragRows) + 32 * g, true);
    }
  }
  long long acc = part;
#pragma unroll
  for (int off = kRows; off < 64; off <<= 1) {
    acc += __shfl_xor(acc, off);
    low |= (uint32_t)__shfl_xor((int)low, off);
  }
  if (lane < kRows) {
    s_sum[wave][lane] = acc;
    s_low[wave][lane] = low;
  }
  __syncthreads();
  if (threadIdx.x < kRows) {
    long long total = 0;
    uint32_t any_low = 0u;
#pragma unroll
    for (int w = 0; w < kFusedWaves; ++w) {
      total += s_sum[w][threadIdx.x];
      any_low |= s_low[w][threadIdx.x];
    }
    sums[m] = total; // a single chunk: K <= kChunkK
    // one-digit row: every value sits in the top digit alone (all-zero and padding rows included)
    shift[m] = bad ? kBadRow : (any_low == 0u ? s + kOneDigitBias : s);
  }
  if (redo.y) {
    // lane rr of every wavefront holds row rr's flag, the same in all wavefronts: the loop is uniform over the block
    const unsigned long long marked = __ballot(bad);
    for (int rr = 0; rr < kRows; ++rr) {
      const int64_t mr = (int64_t)blockIdx.x * kRows + rr;
      if (((marked >> rr) & 1ull) && mr < M)
        redo_marked_row(x + mr * ldx, redo, mr, K, kFusedWaves * 64);
    }
  }
}

template <int kRows, int kPer>
void launch_split_digits_rows(const float *x, int64_t ldx, const float *cs, long long *sums, int32_t *shift,
                              uint4_t *out, int64_t M, int64_t K, const DigitOperand &d, const RowRedo &redo,
                              bool aligned, hipStream_t stream) {
  if (aligned)
    hipLaunchKernelGGL((split_digits_rows<kRows, kPer, true>), dim3((unsigned)(d.rows / kRows)), dim3(kFusedWaves * 64),
                       0, stream, x, ldx, cs, sums, shift, out, M, K, d.k_tiles, d.rows, redo);
  else
    hipLaunchKernelGGL((split_digits_rows<kRows, kPer, false>), dim3((unsigned)(d.rows / kRows)),
                       dim3(kFusedWaves * 64), 0, stream, x, ldx, cs, sums, shift, out, M, K, d.k_tiles, d.rows, redo);
}

// ---- digit operand of a transposed source: the operand's rows are the columns c of src [R, C] (row stride ld) and
// its contraction index runs over src's rows, so x^T, dy^T or W^T feed the digit x digit product without a
// transposed copy.  One scale per column: column maxima by integer atomicMax on the magnitude bits
// (order-independent).
//
// With `detect` the pass also finds out whether every element is zero or a signed power of two no more than six
// binades below its column's largest (INQ weights once they are fixed): then the scale is chosen so that each
// value is an integer of magnitude <= 64 and sits in the lowest digit alone ("narrow" operand, flag word 0), and
// the product needs three digit products instead of six and drops nothing.
__global__ __launch_bounds__(kPrepBlock) void clear_column_scratch(uint32_t *__restrict__ cmax,
                                                                   uint32_t *__restrict__ cmin, int64_t n,
                                                                   int32_t *__restrict__ flag, int flag_value) {
  const int64_t i = (int64_t)blockIdx.x * kPrepBlock + threadIdx.x;
  if (i < n) {
    cmax[i] = 0u;
    cmin[i] = 0xffffffffu;
  }
  if (i == 0)
    *flag = flag_value;
}

// Block = 64 column quads x 4 row groups over a slab of `slab` rows (a multiple of 4); 128-bit loads where the
// layout allows, eight in flight per thread; the row groups are folded through LDS before the atomics.
template <bool kVec, bool kDetect>
__global__ __launch_bounds__(kPrepBlock) void column_absmax(const float *__restrict__ src, int64_t ld, int64_t R,
                                                            int64_t C, uint32_t *__restrict__ cmax,
                                                            uint32_t *__restrict__ cmin, int32_t *__restrict__ flag,
                                                            int slab) {
  __shared__ uint32_t part[4][256];
  __shared__ uint32_t part_min[kDetect ? 4 : 1][256];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + tx) * 4;
  const int64_t r0 = (int64_t)blockIdx.y * slab;
  const int64_t r_end = r0 + slab < R ? r0 + slab : R;
  uint32_t m[4] = {0u, 0u, 0u, 0u}, mn[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  bool other = false; // an element that is neither zero nor a normal power of two
  if (c0 < C) {
#pragma unroll 8
    for (int64_t r = r0 + ty; r < r_end; r += 4) {
      float v[4];
      if (kVec) {
        const float4_t q = *reinterpret_cast<const float4_t *>(src + r * ld + c0);
        v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[j] = (c0 + j < C) ? src[r * ld + c0 + j] : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t u = __float_as_uint(v[j]) & 0x7fffffffu;
        m[j] = u > m[j] ? u : m[j];
        if (kDetect && u) {
          mn[j] = u < mn[j] ? u : mn[j];
          other |= (u & 0x007fffffu) != 0u || (u >> 23) == 0u;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    part[ty][tx * 4 + j] = m[j];
    if (kDetect)
      part_min[ty][tx * 4 + j] = mn[j];
  }
  if (kDetect && __any(other) && (threadIdx.x & 63) == 0 &&
      __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
    atomicOr(flag, 1);
  __syncthreads();
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c < C) {
    uint32_t a = part[0][threadIdx.x], b = part[1][threadIdx.x], d = part[2][threadIdx.x], e = part[3][threadIdx.x];
    a = a > b ? a : b;
    d = d > e ? d : e;
    a = a > d ? a : d;
    if (a)
      atomicMax(&cmax[c], a);
    if (kDetect) {
      a = part_min[0][threadIdx.x], b = part_min[1][threadIdx.x], d = part_min[2][threadIdx.x];
      e = part_min[3][threadIdx.x];
      a = a < b ? a : b;
      d = d < e ? d : e;
      a = a < d ? a : d;
      if (a != 0xffffffffu)
        atomicMin(&cmin[c], a);
    }
  }
}

// Shift of every (padded) operand row from its column maximum; a NaN or an infinity marks the row.  The narrow
// shift (largest element -> 64) replaces the maximum in `cmax`; a column spanning more than six binades raises the
// flag.
__global__ __launch_bounds__(kPrepBlock) void column_shift(uint32_t *__restrict__ cmax,
                                                           const uint32_t *__restrict__ cmin,
                                                           int32_t *__restrict__ shift, int64_t C, int64_t rows,
                                                           int32_t *__restrict__ flag, int detect) {
  const int64_t c = (int64_t)blockIdx.x * kPrepBlock + threadIdx.x;
  if (c >= rows)
    return;
  const uint32_t m = c < C ? cmax[c] : 0u;
  const bool bad = m >= 0x7f800000u;
  shift[c] = bad ? kBadRow : (m == 0u ? 0 : digit_shift(m));
  if (detect) {
    int narrow = 0;
    if (bad) {
      narrow = kBadRow;
    } else if (m != 0u) {
      const int e_max = (int)(m >> 23) - 127, e_min = (int)(cmin[c] >> 23) - 127;
      narrow = 6 - e_max;
      if (e_max - e_min > 6 && __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
        atomicOr(flag, 1);
    }
    cmax[c] = (uint32_t)narrow;
  }
}

// One wavefront per fragment (32 operand rows = columns of src, 32 contraction steps = rows of src); fragments are
// numbered with the column block fastest so that a block's four wavefronts read 512 contiguous bytes of each row.
__global__ __launch_bounds__(kPrepBlock) void split_digits_columns(const float *__restrict__ src, int64_t ld,
                                                                   const int32_t *__restrict__ shift,
                                                                   const int32_t *__restrict__ narrow_shift,
                                                                   const int32_t *__restrict__ flag,
                                                                   uint4_t *__restrict__ out, int64_t R, int64_t C,
                                                                   int64_t k_tiles, int64_t col_blocks,
                                                                   int64_t frags) {
  const int64_t frag = (int64_t)blockIdx.x * (kPrepBlock / 64) + (threadIdx.x >> 6);
  if (frag >= frags)
    return;
  const int lane = threadIdx.x & 63;
  const int64_t mt = frag / col_blocks, cb = frag - mt * col_blocks;
  const int64_t c = cb * kFragRows + (lane & 31);
  const int64_t r0 = mt * kTileK + (lane >> 5) * 16;
  const bool narrow = *flag == 0; // uniform over the grid
  const int s = narrow ? narrow_shift[c] : shift[c];
  const bool live = c < C && s != kBadRow;
  float v[16];
#pragma unroll
  for (int j = 0; j < 16; ++j)
    v[j] = (live && r0 + j < R) ? src[(r0 + j) * ld + c] : 0.0f;
  int q[16];
#pragma unroll
  for (int j = 0; j < 16; ++j)
    q[j] = to_fixed(v[j], s == kBadRow ? 0 : s);
  uint4_t *dst = out + (cb * k_tiles + mt) * kDigits * 64 + lane;
  if (narrow) {
    // every value is a small integer, all of it in the lowest digit: the only fragment a product reads from an
    // operand whose flag is clear
    uint32_t w[3][4];
    pack_digits(q, w);
    uint4_t o;
    o.x = w[kDigits - 1][0], o.y = w[kDigits - 1][1], o.z = w[kDigits - 1][2], o.w = w[kDigits - 1][3];
    __builtin_nontemporal_store(o, dst + (kDigits - 1) * 64);
    return;
  }
  store_digits(q, dst, true);
}

} // namespace

// Digit operand (rows = the C columns of src, contraction over its R rows); `digits` holds
// nbla_hip_digit_operand_bytes(C, R).  The operand's row-sum section serves as scratch (column maxima, then the
// narrow shifts, and the column minima); the digit x digit product does not read row sums.
ColumnScratch column_scratch(void *digits, int64_t R, int64_t C) {
  const DigitOperand d = digit_operand(C, R);
  char *base = static_cast<char *>(digits);
  ColumnScratch s;
  s.cmax = reinterpret_cast<uint32_t *>(base + d.sum_off);
  s.cmin = s.cmax + d.rows;
  s.flag = reinterpret_cast<int32_t *>(base + d.flag_off);
  s.rows = d.rows;
  return s;
}

int launch_split_digits_columns_from_stats(const float *src, int64_t ld, void *digits, int64_t R, int64_t C,
                                           bool detect_narrow, hipStream_t stream) {
  const DigitOperand d = digit_operand(C, R);
  char *base = static_cast<char *>(digits);
  const ColumnScratch cs = column_scratch(digits, R, C);
  int32_t *shift = reinterpret_cast<int32_t *>(base + d.shift_off);
  hipLaunchKernelGGL(column_shift, dim3((unsigned)ceil_div(d.rows, kPrepBlock)), dim3(kPrepBlock), 0, stream, cs.cmax,
                     cs.cmin, shift, C, d.rows, cs.flag, detect_narrow ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("column_shift");
  const int64_t frags = d.k_tiles * d.row_blocks;
  hipLaunchKernelGGL(split_digits_columns, dim3((unsigned)ceil_div(frags, kPrepBlock / 64)), dim3(kPrepBlock), 0,
                     stream, src, ld, shift, reinterpret_cast<const int32_t *>(cs.cmax), cs.flag,
                     reinterpret_cast<uint4_t *>(base), R, C, d.k_tiles, d.row_blocks, frags);
  NBLA_HIP_LAUNCH_CHECK("split_digits_columns");
  return NBLA_HIP_OK;
}

int launch_split_digits_columns(const float *src, int64_t ld, void *digits, int64_t R, int64_t C, bool detect_narrow,
                                hipStream_t stream) {
  const ColumnScratch cs = column_scratch(digits, R, C);
  hipLaunchKernelGGL(clear_column_scratch, dim3((unsigned)ceil_div(cs.rows, kPrepBlock)), dim3(kPrepBlock), 0, stream,
                     cs.cmax, cs.cmin, cs.rows, cs.flag, detect_narrow ? 0 : 1);
  NBLA_HIP_LAUNCH_CHECK("clear_column_scratch");
  int slab = 64; // taller slabs (fewer atomics per column) while a thousand blocks remain
  while (slab < 256 && ceil_div(C, 256) * ceil_div(R, 2 * slab) >= 1024)
    slab *= 2;
  const dim3 grid((unsigned)ceil_div(C, 256), (unsigned)ceil_div(R, slab));
  const bool vec = C % 4 == 0 && ld % 4 == 0 && aligned16(src);
#define NBLA_LAUNCH_ABSMAX(V, D)                                                                                       \
  hipLaunchKernelGGL((column_absmax<V, D>), grid, dim3(kPrepBlock), 0, stream, src, ld, R, C, cs.cmax, cs.cmin,       \
                     cs.flag, slab)
  if (vec && detect_narrow)
    NBLA_LAUNCH_ABSMAX(true, true);
  else if (vec)
    NBLA_LAUNCH_ABSMAX(true, false);
  else if (detect_narrow)
    NBLA_LAUNCH_ABSMAX(false, true);
  else
    NBLA_LAUNCH_ABSMAX(false, false);
#undef NBLA_LAUNCH_ABSMAX
  NBLA_HIP_LAUNCH_CHECK("column_absmax");
  return launch_split_digits_columns_from_stats(src, ld, digits, R, C, detect_narrow, stream);
}

} // namespace nbla_hip


using namespace nbla_hip;

extern "C" {

size_t nbla_hip_packed_bits_bytes(int64_t K, int64_t N) {
  return (size_t)bits_packed_k_tiles(K) * bits_wide_groups(N) * 64 * 4 * sizeof(uint32_t);
}

size_t nbla_hip_digit_operand_bytes(int64_t M, int64_t K) { return digit_operand(M, K).total; }

size_t nbla_hip_binarize_workspace_bytes(int64_t K, int64_t N) {
  const PrepPlan a = make_prep_plan(K, N, false), b = make_prep_plan(K, N, true);
  const size_t wa = a.sums_bytes + a.zeros_bytes + a.pairs_bytes, wb = b.sums_bytes + b.zeros_bytes + b.pairs_bytes;
  return wa > wb ? wa : wb;
}

int nbla_hip_binarize_weights_f32(const float *W, float *Wb, float *alpha, uint32_t *bits, int64_t K, int64_t N,
                                  int transposed, float quantize_zero_to, int *zero_count, void *workspace,
                                  size_t workspace_bytes, void *stream_) {
  if (K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "weight matrix must not be empty (K=%lld, N=%lld).", (long long)K, (long long)N);
  const PrepPlan P = make_prep_plan(K, N, transposed != 0);
  if (workspace_bytes < P.sums_bytes + P.zeros_bytes + P.pairs_bytes || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "binarize workspace too small or misaligned.");
  if (!aligned16(bits))
    return fail(NBLA_HIP_ERR_MEMORY, "packed-bit buffer must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  float *sums = static_cast<float *>(workspace);
  int *zeros = reinterpret_cast<int *>(static_cast<char *>(workspace) + P.sums_bytes);
  uint32_t *pairs = reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + P.sums_bytes + P.zeros_bytes);
  int64_t slices = P.slices;
  if (!transposed) {
    if (P.slabs <= 65535 && (uint64_t)N * 4 < (1ull << 32)) {
      // a lane's four columns as one 128-bit access where the rows allow it (a null Wb -- no fp32 signs wanted --
      // counts as aligned), else as four 32-bit ones
      const bool aligned = N % 4 == 0 && N >= 4 && aligned16(W) && aligned16(Wb);
      // writes the packed operand itself (padding k tiles included): nothing is left for the relayout below
      // fewer than four blocks per CU with 256-row slabs: halve the slabs
      const bool fine = P.wide_groups * P.slabs < 1024 && 2 * P.slabs <= 65535;
      const int64_t slabs = fine ? 2 * P.slabs : P.slabs;
      const dim3 grid((unsigned)P.wide_groups, (unsigned)slabs);
      uint4_t *packed = reinterpret_cast<uint4_t *>(bits);
#define NBLA_BINARIZE_WIDE(ROWS, COUNT)                                                                                \
  do {                                                                                                                 \
    if (aligned)                                                                                                       \
      hipLaunchKernelGGL((binarize_kn_wide<ROWS, COUNT, true>), grid, dim3(kPrepBlock), 0, stream, W, Wb, packed, sums,  \
                         zeros, K, N, P.wide_groups, P.Npw, quantize_zero_to);                                         \
    else                                                                                                               \
      hipLaunchKernelGGL((binarize_kn_wide<ROWS, COUNT, false>), grid, dim3(kPrepBlock), 0, stream, W, Wb, packed, sums, \
                         zeros, K, N, P.wide_groups, P.Npw, quantize_zero_to);                                         \
  } while (0)
      if (fine && zero_count)
        NBLA_BINARIZE_WIDE(32, true);
      else if (fine)
        NBLA_BINARIZE_WIDE(32, false);
      else if (zero_count)
        NBLA_BINARIZE_WIDE(64, true);
      else
        NBLA_BINARIZE_WIDE(64, false);
#undef NBLA_BINARIZE_WIDE
      NBLA_HIP_LAUNCH_CHECK("binarize_kn_wide");
      if (alpha || zero_count) {
        hipLaunchKernelGGL(binarize_finalize, dim3((unsigned)ceil_div(N, kPrepBlock)), dim3(kPrepBlock), 0, stream, sums,
                           zeros, alpha, zero_count, N, P.Npw, slabs, slabs * P.wide_groups, (float)1 / K, pairs,
                           reinterpret_cast<uint4_t *>(bits), P.k_tiles, P.col_groups, P.wide_groups, (int64_t)0);
        NBLA_HIP_LAUNCH_CHECK("binarize_finalize");
      }
      return NBLA_HIP_OK;
    } else {
      slices = ceil_div(K, kKSlice);
      const dim3 grid((unsigned)P.col_groups, (unsigned)slices);
      hipLaunchKernelGGL(binarize_kn<false>, grid, dim3(kPrepBlock), 0, stream, W, Wb, pairs, sums, zeros, K, N,
                         P.col_groups, P.Np, quantize_zero_to);
    }
  } else {
    if (P.col_groups <= 65535 && K % 4 == 0 && aligned16(W) && aligned16(Wb)) {
      hipLaunchKernelGGL(binarize_nk_vec<true>, dim3((unsigned)P.slices, (unsigned)P.col_groups), dim3(kPrepBlock), 0,
                         stream, W, Wb, pairs, sums, zeros, K, N, P.col_groups, P.Np, P.k_tiles, quantize_zero_to);
    } else if (P.col_groups <= 65535) {
      hipLaunchKernelGGL(binarize_nk_vec<false>, dim3((unsigned)P.slices, (unsigned)P.col_groups), dim3(kPrepBlock), 0,
                         stream, W, Wb, pairs, sums, zeros, K, N, P.col_groups, P.Np, P.k_tiles, quantize_zero_to);
    } else {
      const dim3 grid((unsigned)P.col_groups, (unsigned)P.slices);
      hipLaunchKernelGGL(binarize_nk, grid, dim3(kPrepBlock), 0, stream, W, Wb, pairs, sums, zeros, K, N, P.col_groups,
                         P.Np, P.k_tiles, quantize_zero_to);
    }
  }
  NBLA_HIP_LAUNCH_CHECK("binarize_weights");
  {
    const int64_t wide_groups = bits_wide_groups(N), total = bits_packed_k_tiles(K) * wide_groups * 64;
    const float inv_k = (float)1 / K;
    const int64_t threads = total > N ? total : N;
    hipLaunchKernelGGL(binarize_finalize, dim3((unsigned)ceil_div(threads, kPrepBlock)), dim3(kPrepBlock), 0, stream,
                       sums, zeros, alpha, zero_count, N, P.Np, slices, slices * P.col_groups, inv_k, pairs,
                       reinterpret_cast<uint4_t *>(bits), P.k_tiles, P.col_groups, wide_groups, total);
    NBLA_HIP_LAUNCH_CHECK("binarize_finalize");
  }
  return NBLA_HIP_OK;
}

int nbla_hip_split_digits_f32(const float *x, int64_t ldx, void *xdigits, int64_t M, int64_t K, void *stream_) {
  return nbla_hip_split_digits_scaled_f32(x, ldx, nullptr, xdigits, M, K, stream_);
}

int nbla_hip_split_digits_scaled_f32(const float *x, int64_t ldx, const float *colscale, void *xdigits, int64_t M,
                                     int64_t K, void *stream_) {
  return launch_split_digits_rows_redo(x, ldx, colscale, xdigits, M, K, nullptr, nullptr, as_stream(stream_));
}

} // extern "C"

namespace nbla_hip {

int launch_split_digits_rows_redo(const float *x, int64_t ldx, const float *colscale, void *xdigits, int64_t M,
                                  int64_t K, const RowRedo *redo_in, bool *redone, hipStream_t stream) {
  const float *cs = colscale;
  const RowRedo redo = (redo_in && !colscale) ? *redo_in : RowRedo{nullptr, nullptr, nullptr, nullptr, 0};
  if (redone)
    *redone = false;
  if (M <= 0 || K <= 0 || ldx < K)
    return fail(NBLA_HIP_ERR_VALUE, "invalid digit operand shape (M=%lld, K=%lld, ldx=%lld).", (long long)M,
                (long long)K, (long long)ldx);
  if (!aligned16(xdigits))
    return fail(NBLA_HIP_ERR_MEMORY, "digit operand buffer must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  const DigitOperand d = digit_operand(M, K);
  char *base = static_cast<char *>(xdigits);
  long long *sums = reinterpret_cast<long long *>(base + d.sum_off);
  int32_t *shift = reinterpret_cast<int32_t *>(base + d.shift_off);
  const bool vec = K % 4 == 0 && ldx % 4 == 0 && aligned16(x) && aligned16(cs);
  if (d.k_tiles <= 512) { // rows of up to 16384 values: one pass, rows held in registers
    uint4_t *out = static_cast<uint4_t *>(xdigits);
    // A block covers 8 wavefronts x (32 / rows) x (tiles per lane) k tiles.  Most rows per block (longest store runs)
    // among the shapes that hold the row and still give every CU a block; the fewest rows otherwise.
    const int64_t kt = d.k_tiles;
    int rows_per_block = 0;
    for (int rows : {16, 8, 4}) {
      const int64_t per = ceil_div(kt, kFusedWaves * (32 / rows));
      if (per > (rows == 8 ? 11 : 8))
        continue;
      rows_per_block = rows;
      if (d.rows / rows >= 256)
        break;
    }
    const int64_t per = ceil_div(kt, kFusedWaves * (32 / rows_per_block));
#define NBLA_SPLIT_ROWS(R, P)                                                                                          \
  launch_split_digits_rows<R, P>(x, ldx, cs, sums, shift, out, M, K, d, redo, vec, stream)
    if (rows_per_block == 16) {
      if (per <= 1)
        NBLA_SPLIT_ROWS(16, 1);
      else if (per <= 2)
        NBLA_SPLIT_ROWS(16, 2);
      else if (per <= 4)
        NBLA_SPLIT_ROWS(16, 4);
      else
        NBLA_SPLIT_ROWS(16, 8);
    } else if (rows_per_block == 8) {
      if (per <= 1)
        NBLA_SPLIT_ROWS(8, 1);
      else if (per <= 2)
        NBLA_SPLIT_ROWS(8, 2);
      else if (per <= 4)
        NBLA_SPLIT_ROWS(8, 4);
      else if (per <= 6)
        NBLA_SPLIT_ROWS(8, 6);
      else if (per <= 8)
        NBLA_SPLIT_ROWS(8, 8);
      else
        NBLA_SPLIT_ROWS(8, 11);
    } else {
      if (per <= 1)
        NBLA_SPLIT_ROWS(4, 1);
      else if (per <= 2)
        NBLA_SPLIT_ROWS(4, 2);
      else if (per <= 4)
        NBLA_SPLIT_ROWS(4, 4);
      else if (per <= 6)
        NBLA_SPLIT_ROWS(4, 6);
      else
        NBLA_SPLIT_ROWS(4, 8);
    }
#undef NBLA_SPLIT_ROWS
    NBLA_HIP_LAUNCH_CHECK("split_digits_rows");
    if (redone)
      *redone = redo.y != nullptr;
    return NBLA_HIP_OK;
  }
  const dim3 scale_grid((unsigned)ceil_div(d.rows, kPrepBlock / 64));
  if (vec)
    hipLaunchKernelGGL(digit_row_scale<true>, scale_grid, dim3(kPrepBlock), 0, stream, x, ldx, cs, sums, shift, M, K,
                       d.rows, d.chunks);
  else
    hipLaunchKernelGGL(digit_row_scale<false>, scale_grid, dim3(kPrepBlock), 0, stream, x, ldx, cs, sums, shift, M, K,
                       d.rows, d.chunks);
  NBLA_HIP_LAUNCH_CHECK("digit_row_scale");
  const int64_t frags = d.row_blocks * d.k_tiles;
  if (K % 64 == 0 && ldx % 4 == 0 && aligned16(x) && aligned16(cs)) {
    const int64_t patches = frags / 2;
    hipLaunchKernelGGL(split_digits_tiled, dim3((unsigned)ceil_div(patches, kPrepBlock / 64)), dim3(kPrepBlock), 0,
                       stream, x, ldx, cs, shift, static_cast<uint4_t *>(xdigits), M, K, d.k_tiles, patches);
  } else {
    hipLaunchKernelGGL(split_digits, dim3((unsigned)ceil_div(frags, kPrepBlock / 64)), dim3(kPrepBlock), 0, stream, x,
                       ldx, cs, shift, static_cast<uint4_t *>(xdigits), M, K, d.k_tiles, frags);
  }
  NBLA_HIP_LAUNCH_CHECK("split_digits");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
