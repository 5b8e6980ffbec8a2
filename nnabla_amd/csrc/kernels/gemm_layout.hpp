// Operand layouts shared by the kernels that produce GEMM operands (sign
// binarisation, bf16x3 split, im2col, INQ) and the MFMA kernels that consume
// them.
//
// The contraction is y[m, n] = sum_k A[m, k] * B[k, n] on
// v_mfma_f32_32x32x16_bf16.  One MFMA operand fragment covers 32 rows (m for
// A, n for B) by 16 k; lane l of the wavefront holds row (l % 32) and the eight
// k values (l / 32) * 8 + 0..7, i.e. 16 bytes of bf16.
//
// A ("split operand"): an fp32 matrix is stored as three bf16 planes
// hi/mid/lo with x == hi + mid + lo exactly, already in fragment order:
//     A'[row_block = m / 32][k_block = k / 16][plane][lane][8 x bf16]
// so a fragment is 1 KiB of consecutive bytes, read by lane l at offset 16 * l.
// Rows >= M and columns >= K are zero.  K is padded to a multiple of 32 (two
// k blocks: one kernel k-step), M to a multiple of 32.
//
// B ("packed bits"): one bit per weight, set = negative (-1), clear = +1:
//     B'[k_tile = k / 32][col_group = n / 64][lane] : one uint32 word
// Lane l's word serves column n = col_group * 64 + f * 32 + (l % 32) for
// f = 0, 1 and k = k_tile * 32 + s * 16 + (l / 32) * 8 + e for s = 0, 1 and
// e = 0..7.  With j = 2 f + s, i = e / 2 and p = 4 j + i the bit sits at
// position 15 - p (e even) or 31 - p (e odd), so that
//     ((word << p) & 0x80008000) | 0x3F803F80
// is directly the register holding the bf16 pair (+-1.0, +-1.0) for k = e, e+1
// of fragment (f, s).  Bits outside [K, N] are clear.
#pragma once
#include <stdint.h>

namespace nbla_hip {

constexpr int kFragRows = 32;   // rows per MFMA fragment
constexpr int kFragK = 16;      // k per MFMA fragment
constexpr int kTileK = 32;      // k per kernel step (two fragments)
constexpr int kColGroup = 64;   // columns per packed word group
constexpr int kFragBytes = 1024;

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

__host__ __device__ inline int64_t split_row_blocks(int64_t M) { return ceil_div(M, kFragRows); }
__host__ __device__ inline int64_t split_k_blocks(int64_t K) { return ceil_div(K, kTileK) * 2; }
__host__ __device__ inline int64_t bits_k_tiles(int64_t K) { return ceil_div(K, kTileK); }
__host__ __device__ inline int64_t bits_col_groups(int64_t N) { return ceil_div(N, kColGroup); }

// Bit position inside a packed word for fragment (f, s) and k-offset e.
__host__ __device__ inline int packed_bit_position(int f, int s, int e) {
  const int p = 4 * (2 * f + s) + (e >> 1);
  return (e & 1) ? 31 - p : 15 - p;
}

} // namespace nbla_hip
