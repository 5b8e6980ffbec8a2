// Operand layouts shared by the kernels that produce GEMM operands (sign binarisation, digit split, im2col, INQ) and
// the MFMA kernels that consume them.
//
// The contraction is y[m, n] = sum_k A[m, k] * B[k, n] on v_mfma_i32_32x32x32_i8.  One i8 operand fragment covers
// 32 rows (m for A, n for B) by 32 k; lane l holds row (l % 32) and sixteen bytes, byte j being k-slot
// (l / 32) * 16 + j of the k tile: a fragment is 1 KiB of consecutive bytes, read by lane l at offset 16 * l.
//
// X ("digit operand"): row m of an fp32 matrix is turned into integers q = rint(x * 2^s_m), |q| < 2^23, with one
// power-of-two scale per row (s_m the largest shift that keeps the row's largest magnitude inside the digit range),
// and q into three balanced base-256 digits q = d0 * 65536 + d1 * 256 + d2, each an int8:
//     X'[row_block = m / 32][k_tile = k / 32][digit 0..2][lane][16 x int8]
// followed, per chunk of kChunkK columns, by the row sums of q (one int64 array of row_blocks * 32 entries per
// chunk), by the shifts s_m (one int32 array; kBadRow marks a row holding a non-finite value) and by a 256-byte tail
// whose first word is the mode flag of column-scaled operands (0: every row is held in its lowest digit alone).
// Rows >= M and columns >= K are zero.  The number of k tiles is padded to a multiple of 8.
//
// B ("packed bits"): one bit per weight, set = negative (-1), clear = +1, in groups of 256 columns (eight column
// fragments F = 0..7 of 32 columns):
//     B'[k_tile = k / 32][wide_group = n / 256][lane][4 x uint32]
// Word i (0..3) of lane l serves column n = wide_group * 256 + F * 32 + (l % 32) and k-slots (l / 32) * 16 + 4 i + c,
// c = 0..3; the bit of (F, c) sits at position F + 8 c, so that
//     word_i & (0x01010101 << F)
// is directly register i of the i8 fragment of column fragment F, holding 2^F (as int8: -128 for F = 7) for a
// negative weight and 0 otherwise: the accumulators of fragment F come out scaled by that constant, which the
// epilogue divides out exactly.  With b in {0, 1} the signed product is  sum q * (1 - 2 b) = rowsum(q) - 2 sum q b.
// Bits outside [K, N] are clear; the number of k tiles is padded to a multiple of 8.
//
// The kernels that binarise weights first emit "pair words" (an intermediate kept in their workspace):
//     P[k_tile][pair_group = n / 64][lane] : one uint32, bit 4 f + j / 4 + 8 (j % 4) for column half f = 0, 1 and
//     k-slot offset j = 0..15 of the lane
// and a small relayout pass interleaves four pair groups into one wide group.
#pragma once
#include <stdint.h>

namespace nbla_hip {

constexpr int kFragRows = 32;   // rows per MFMA fragment
constexpr int kTileK = 32;      // k per i8 MFMA fragment and k tile
constexpr int kColGroup = 64;   // columns per pair-word group
constexpr int kFragBytes = 1024;

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

__host__ __device__ inline int64_t split_row_blocks(int64_t M) { return ceil_div(M, kFragRows); }
__host__ __device__ inline int64_t bits_k_tiles(int64_t K) { return ceil_div(K, kTileK); }
__host__ __device__ inline int64_t bits_col_groups(int64_t N) { return ceil_div(N, kColGroup); }

// Bit position inside a pair word for column half f and k-slot offset j (0..15) of the lane.
__host__ __device__ inline int packed_bit_position(int f, int j) { return 4 * f + (j >> 2) + 8 * (j & 3); }

constexpr int kWideGroup = 256; // columns per group of the packed operand
__host__ __device__ inline int64_t bits_wide_groups(int64_t N) { return ceil_div(N, kWideGroup); }
// k tiles of the packed operand: padded like the digit operand's, the padding tiles all clear
__host__ __device__ inline int64_t bits_packed_k_tiles(int64_t K) { return ceil_div(K, 8 * kTileK) * 8; }

// ---- digit operand geometry
constexpr int kDigits = 3;
constexpr int64_t kChunkK = 16384;        // columns whose i32 accumulators are folded together (keeps them < 2^31)
constexpr int kDigitMax = 8355711;        // 127 * 65536 + 127 * 256 + 127: the largest q three balanced digits hold
constexpr int kBadRow = -2147483647 - 1;  // shift value marking a row with a NaN or an infinity
// A row whose values all have zero lower digits d1 = d2 = 0 under the row's ordinary scale is a "one-digit row": this
// is what rows of small fixed-point numbers look like (outputs of a fixed-point quantizer: multiples of one power of
// two, at most seven bits from the unit to the largest magnitude -- the scale puts the largest magnitude into the top
// digit and every other value is a whole number of top-digit units).  The producer marks such a row by storing its
// shift with kOneDigitBias added (plain shifts lie in [-105, 171]); a product whose tile holds only such rows skips
// the lower digits' fragments.  Nothing else changes -- digits, scale and row sums are the ordinary ones -- so both
// forms of the product give the same bits.
constexpr int kOneDigitBias = 1024;
__host__ __device__ inline bool one_digit_row(int shift) { return shift >= kOneDigitBias / 2; }
__host__ __device__ inline int plain_shift(int shift) { return one_digit_row(shift) ? shift - kOneDigitBias : shift; }

// k tiles of both bit-weight operands are padded (with zeros) to a multiple of 8: a kernel k step is two tiles and
// a block may split the contraction over four wavefront groups
__host__ __device__ inline int64_t digit_k_tiles(int64_t K) { return ceil_div(K, 8 * kTileK) * 8; }
__host__ __device__ inline int64_t digit_chunks(int64_t K) { return ceil_div(K, kChunkK); }
// byte offsets of the sections of a digit operand
struct DigitOperand {
  int64_t row_blocks, k_tiles, rows, chunks;
  size_t sum_off, shift_off, flag_off, total;
};
__host__ __device__ inline DigitOperand digit_operand(int64_t M, int64_t K) {
  DigitOperand d;
  d.row_blocks = split_row_blocks(M);
  d.k_tiles = digit_k_tiles(K);
  d.rows = d.row_blocks * kFragRows;
  d.chunks = digit_chunks(K);
  d.sum_off = (size_t)d.row_blocks * d.k_tiles * kDigits * kFragBytes;
  d.shift_off = d.sum_off + (size_t)d.chunks * d.rows * sizeof(int64_t);
  d.flag_off = d.shift_off + (size_t)d.rows * sizeof(int32_t); // one word: see launch_split_digits_columns
  d.total = d.flag_off + 256;
  return d;
}

#if defined(__HIPCC__)
// Sixteen fixed-point values q (|q| <= kDigitMax) of one lane -> its four words of each digit fragment (digit 0 the
// top one; value j in byte j % 4 of word j / 4).  The three balanced base-256 digits of q are the low three bytes of
// q + 0x808080, each with its top bit flipped: adding 128 per digit position makes every digit a plain byte, and the
// carries between the positions are exactly the borrows of the balanced form.  Four values' digits are then
// transposed into one word per digit with byte permutes.
__device__ __forceinline__ void pack_digits(const int (&q)[16], uint32_t (&w)[3][4]) {
#pragma unroll
  for (int g4 = 0; g4 < 4; ++g4) {
    uint32_t d[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      d[j] = ((uint32_t)q[4 * g4 + j] + 0x808080u) ^ 0x808080u; // bytes: lowest, middle, top digit, unused
    const uint32_t t01 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u); // d0.b0 d1.b0 d0.b1 d1.b1
    const uint32_t t23 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
    const uint32_t u01 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u); // d0.b2 d1.b2 d0.b3 d1.b3
    const uint32_t u23 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
    w[2][g4] = __builtin_amdgcn_perm(t23, t01, 0x05040100u); // lowest digits
    w[1][g4] = __builtin_amdgcn_perm(t23, t01, 0x07060302u); // middle digits
    w[0][g4] = __builtin_amdgcn_perm(u23, u01, 0x05040100u); // top digits
  }
}

// Blocks are handed to the 8 XCDs round-robin; give each XCD a contiguous run
// of tiles (n fastest) so that blocks resident on one XCD share an X panel in
// that XCD's L2.
__device__ __forceinline__ int64_t xcd_remap(int64_t b, int64_t total) {
  constexpr int64_t kXcds = 8;
  const int64_t per = total / kXcds, rem = total % kXcds;
  const int64_t xcd = b % kXcds, slot = b / kXcds;
  // XCDs [0, rem) own per+1 tiles, the rest own per tiles.
  const int64_t start = xcd * per + (xcd < rem ? xcd : rem);
  return start + slot;
}

// Tile (bm, bn) of block b: an XCD's run of tiles is walked in bands of kBand tile rows, column by column inside a
// band, so the blocks resident on an XCD at one time cover a compact patch of tiles and its L2 serves each row
// panel and each column panel to several of them.
template <int kBand>
__device__ __forceinline__ void band_tile(int64_t b, int64_t blocks_m, int64_t blocks_n, int64_t &bm, int64_t &bn) {
  const int64_t tile = xcd_remap(b, blocks_m * blocks_n);
  const int64_t band = tile / (kBand * blocks_n), in_band = tile - band * (kBand * blocks_n);
  const int64_t band_rows = (blocks_m - band * kBand < kBand) ? blocks_m - band * kBand : kBand;
  bn = in_band / band_rows;
  bm = band * kBand + (in_band - bn * band_rows);
}
#endif

} // namespace nbla_hip
