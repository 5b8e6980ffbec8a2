// BinaryWeightAffine / BinaryConnectAffine forward for some hundreds of input rows (65 <= M <= 512), in ONE walk over
// W: the pass that writes Sign(W) and sums |W| per column also multiplies, on the int8 matrix cores.
//
// At these row counts the forward is still bound by the weights (4 B read and 4 B written per weight; the fp32 signs
// Wb are an output of the function), but the product is too large for one wavefront's registers.  The general path
// pays for that with two walks (binarise W to packed bits, then multiply them).  Here a block of eight wavefronts owns
// a 128-column strip of W (over all of K, or over one of a few slices of K when the strips alone would leave CUs
// empty) and a chunk of up to 256 rows of x:
//   * four "weight" wavefronts stream the strip through an LDS ring (global -> LDS copies, kRingDepth k steps of
//     32 rows ahead);
//   * four "activation" wavefronts copy the k step's digit fragments of x (the operand split_digits_rows writes: three
//     balanced base-256 digits per value, one power-of-two scale per row) into a double-buffered LDS stage;
//   * all eight wavefronts convert -- each takes four of the k step's 32 rows, turns every weight into its sign,
//     stores Wb, adds |w| to its column sums and leaves the signs in LDS as the B fragments of
//     v_mfma_i32_32x32x32_i8: byte +64 or -64, so an accumulator holds 64 sum_k q s exactly -- and multiply:
//     wavefront w owns rows 32 w .. 32 w + 31 and all 128 columns of the 256 x 128 output tile, three int32
//     accumulator sets (192 registers), 12 MFMAs per k step.
// What the shape answers to, per k step and CU: 12 x 8 MFMAs = 768 cycles of the matrix pipes; 40 KiB entering
// through the vector memory path (24 digits + 16 weights; a 512 x 64 tile moved 56); about 110 KiB of LDS traffic;
// and the vector instructions of the conversion, which on a SIMD ADD to the time of its MFMAs (measured: matrix pipes
// 35 % and vector ALUs 43 % busy at 119 vector instructions per wavefront and k step, the rest waits), so everything
// that is not an MFMA is kept off the vector ALUs: signs are the sign bit over 1.0 (a select only in k steps where some
// lane holds a zero or a NaN), the fragments hold bytes that need no expansion, row offsets travel in scalar
// registers.  A lone wavefront issues one instruction every ten cycles or so, so the conversion is spread over all
// wavefronts, and the two wavefronts of a SIMD (w and w + 4) run conversion and multiplication in opposite orders.
// The two copying roles keep separate memory counters: a wavefront's vmcnt retires in order, so a wavefront that waits
// for the digits it asked for two k steps ago would also drain its weight copies, which must stay in flight for
// several k steps to cover HBM latency.  One workgroup barrier per k step hands the bit tile, the weights that have
// landed and the digit stage over.
// With more than 256 rows two blocks (row chunks) walk the same strip; they run on the same XCD, one behind the other
// in dispatch order, so the second finds the strip in that XCD's L2.  Only chunk 0 stores Wb and alpha.
//
// Epilogue: the wavefronts' column sums are folded in a fixed order, alpha = colsum * ((float)1 / K)
// (binary_weight_affine.cpp:68), and y = (sum_k q s) * 2^-shift * alpha + bias, the integer sum combined from the
// three accumulators exactly and rounded once.  With K in slices, a block stores its fp32 partial products and column
// sums instead and a second launch adds the slices in slice order.
// Rows of x that hold a NaN or an infinity are left to the caller (affine_redo_marked_rows).  Sign(0) =
// quantize_zero_to other than +-1 cannot be a sign byte: the walk raises a flag when it meets such a weight and the
// caller's fp32 product (which runs only when the flag is up) replaces y.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kStripCols = 128;                     // columns of W per block: four column fragments
constexpr int kChunkRows = 256;                     // rows of x per block: eight row fragments
constexpr int kRowFrags = kChunkRows / kFragRows;
constexpr int kRowsThreads = 512;                   // eight wavefronts
constexpr int kRingDepth = 5;                       // k steps of W in flight ahead of the one being converted
constexpr int kRingSlots = kRingDepth + 1;
constexpr int kRawBytes = kTileK * kStripCols * 4;  // one k step of the strip as fp32: 16 KiB
constexpr int kBTileBytes = 4 * kFragBytes;         // the signs of one k step: four column fragments of bytes
constexpr int kAStages = 2;
constexpr int kAStageBytes = kRowFrags * kDigits * kFragBytes; // 24 KiB
constexpr int kALoads = kRowFrags * kDigits / 4;    // fragment copies per activation wavefront and k step
constexpr int kWLoads = 4;                          // copies per weight wavefront and k step
constexpr int kConvStores = 4;                      // Wb stores per wavefront and k step (four rows, two columns each)
constexpr int kRingOff = kAStages * kAStageBytes;
constexpr int kBOff = kRingOff + kRingSlots * kRawBytes;
constexpr int kRowsLdsBytes = kBOff + 2 * kBTileBytes;
static_assert(kRowsLdsBytes <= 160 * 1024, "the stages fit the CU's LDS");
static_assert((kWLoads + kConvStores) * kRingDepth <= 63 && kALoads + kConvStores <= 63, "vmcnt is a 6-bit counter");
constexpr int kSignScaleLog2 = 6;                   // sign bytes are +-64
static_assert(kChunkK * 128 * 64 < (1ll << 31), "64 x digit sums of a chunk of K fit the int32 accumulators");

struct RowsArgs {
  const float *W;
  float *Wb;
  const uint4_t *xd;     // digit fragments of x
  const int32_t *shift;  // per-row scale exponents
  float *alpha;          // may be null (BinaryConnect)
  const float *bias;     // may be null
  float *y;
  float *partial;        // K in slices: [slices][M][N] partial products, then [slices][N] column sums
  int *zero_flag;        // raised when a weight is neither negative nor positive and zero_to is not +-1 (may be null)
  int64_t M, K, N;
  int64_t row_blocks, x_k_tiles;
  int ksteps;            // ceil(K / 32)
  int strips, chunks, slices, slice_steps;
  float zero_to, inv_k;
};

// sign.hpp:48-50
// (w > 0 ? 1 : (w < 0 ? -1 : zero_to): the sign bit over 1.0 unless w is a zero or a NaN)

#define NBLA_ROWS_BARRIER()                                                                                            \
  do {                                                                                                                 \
    asm volatile("" ::: "memory");                                                                                     \
    __builtin_amdgcn_s_barrier();                                                                                      \
    asm volatile("" ::: "memory");                                                                                     \
  } while (0)
// vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
#define NBLA_ROWS_WAIT_VMCNT(n)                                                                                        \
  do {                                                                                                                 \
    asm volatile("" ::: "memory");                                                                                     \
    __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8));                            \
    asm volatile("" ::: "memory");                                                                                     \
  } while (0)
#define NBLA_ROWS_WAIT_LGKM0()                                                                                         \
  do {                                                                                                                 \
    asm volatile("" ::: "memory");                                                                                     \
    __builtin_amdgcn_s_waitcnt(0xc07f);                                                                                \
    asm volatile("" ::: "memory");                                                                                     \
  } while (0)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_rsrc(const void *p, uint32_t bytes) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint64_t u = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(u), 0, __builtin_amdgcn_readfirstlane((int)bytes),
                                           0x00020000);
}

__global__ __launch_bounds__(kRowsThreads, 1) void binary_affine_rows_kernel(RowsArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  typedef __attribute__((address_space(3))) void lds_void_t;
  constexpr int D = kRingDepth;

  // Blocks are handed to the eight XCDs round-robin.  Block index = ((strip / 8 * slices + slice) * chunks + chunk)
  // * 8 + strip % 8: the row chunks of one strip and slice follow each other on one XCD.
  int q = blockIdx.x >> 3;
  const int chunk = q % a.chunks;
  q /= a.chunks;
  const int slice = q % a.slices;
  const int strip = (q / a.slices) * 8 + (blockIdx.x & 7);
  if (strip >= a.strips)
    return;
  const int t_begin = slice * a.slice_steps;
  const int T = (a.ksteps - t_begin < a.slice_steps) ? a.ksteps - t_begin : a.slice_steps; // k steps of this block

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool weights = wave >= 4; // role of this wavefront
  const int v = wave & 3;
  const int64_t n0 = (int64_t)strip * kStripCols;
  const int64_t m0 = (int64_t)chunk * kChunkRows;
  const uint32_t row_bytes = (uint32_t)(a.N * 4);
  const uint32_t step_bytes = row_bytes * kTileK;

  i32x16_t acc[kDigits][4];
#pragma unroll
  for (int d = 0; d < kDigits; ++d)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[d][j][r] = 0;

  // ---- weight wavefronts: the strip as a buffer that starts at its first column; reads past the end of W (k steps
  // beyond K, issued to keep the counters uniform) give zeros, stores past it are dropped (the range check covers the
  // scalar offset as well as the lane's).
  const uint32_t strip_bytes = (uint32_t)((a.K * a.N - n0) * 4);
  const __amdgpu_buffer_rsrc_t w_rsrc = rows_rsrc(a.W + n0, strip_bytes);
  const __amdgpu_buffer_rsrc_t wb_rsrc = rows_rsrc(a.Wb + n0, strip_bytes);
  // copy p (0..3) of weight wavefront v: lane l fetches 16 bytes of row 8 v + 2 p + l / 32 at columns 4 (l % 32) ..
  uint32_t w_off = (uint32_t)(t_begin * kTileK + 8 * v + (lane >> 5)) * row_bytes + (uint32_t)(lane & 31) * 16u;
  uint32_t row_soff[4]; // 0, 1, 2, 3 (conversion) x row; twice that for the copies
#pragma unroll
  for (int r = 0; r < 4; ++r)
    row_soff[r] = __builtin_amdgcn_readfirstlane((int)(r * row_bytes));
  // conversion: wavefront w takes rows 4 w .. 4 w + 3 of a k step, lane = column pair 2 l, 2 l + 1 of the strip (both
  // inside W or both outside: N % 4 == 0).  Only row chunk 0 stores Wb, the others send theirs past the end.
  const bool col_ok = n0 + 2 * lane < a.N;
  uint32_t wb_off =
      (col_ok && chunk == 0) ? (uint32_t)(t_begin * kTileK + 4 * wave) * row_bytes + (uint32_t)lane * 8u : 0x80000000u;
  int ring_next = 0; // ring slot (bytes) of the next copy
  int ring_conv = 0; // ring slot of the next conversion
  auto issue_w = [&]() __attribute__((always_inline)) {
    unsigned char *dst = smem + kRingOff + ring_next + v * 4096;
    static_assert(kWLoads == 4, "one copy per pair of rows");
#pragma unroll
    for (int p = 0; p < 4; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_void_t *)(dst + p * 1024), 16, w_off, 2 * row_soff[p], 0, 0);
    w_off += step_bytes;
    ring_next = (ring_next + kRawBytes == kRingSlots * kRawBytes) ? 0 : ring_next + kRawBytes;
  };
  float2_t colsum = {0.0f, 0.0f};
  // Lanes that have met a weight which is neither negative nor positive (a zero or a NaN: Sign gives zero_to), as a
  // wavefront mask.  Rows past K read as zeros and are left out; they only occur in the last k step.
  uint64_t special = 0;
  int rows_left = (int)a.K - (t_begin * kTileK + 4 * wave); // rows of W from this wavefront's first row of the next conversion on
  const uint32_t zero_to_bits = __float_as_uint(a.zero_to);
  // rows 4 w .. 4 w + 3 of the k step in ring slot ring_conv -> Wb, column sums, B tile `b_bytes`
  auto convert = [&](int b_bytes) __attribute__((always_inline)) {
    const float2_t *raw = reinterpret_cast<const float2_t *>(smem + kRingOff + ring_conv + wave * 2048) + lane;
    float2_t w[4];
    uint32_t s[2][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
      w[r] = raw[r * (kStripCols / 2)];
    // the sign bit over 1.0: right for every weight that is negative or positive
    uint64_t odd = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[0][r] = (__float_as_uint(w[r].x) & 0x80000000u) | 0x3f800000u;
      s[1][r] = (__float_as_uint(w[r].y) & 0x80000000u) | 0x3f800000u;
      const uint64_t m = __builtin_amdgcn_ballot_w64(!__builtin_islessgreater(w[r].x, 0.0f)) |
                         __builtin_amdgcn_ballot_w64(!__builtin_islessgreater(w[r].y, 0.0f));
      odd |= (r < rows_left) ? m : 0; // (uniform)
      colsum.x += fabsf(w[r].x);
      colsum.y += fabsf(w[r].y);
    }
    if (odd != 0) { // uniform, and rare: some lane holds a zero or a NaN
      special |= odd;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[0][r] = __builtin_islessgreater(w[r].x, 0.0f) ? s[0][r] : zero_to_bits;
        s[1][r] = __builtin_islessgreater(w[r].y, 0.0f) ? s[1][r] : zero_to_bits;
      }
    }
    rows_left -= kTileK;
    static_assert(kConvStores == 4, "one store per row");
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      uint2_t o;
      o.x = s[0][r], o.y = s[1][r];
      __builtin_amdgcn_raw_buffer_store_b64(o, wb_rsrc, wb_off, row_soff[r], 2);
    }
    wb_off += step_bytes; // (0x80000000 + at most 2^31 - 1: stays past the end)
    // B fragments: column c of the strip is lane c % 32 of fragment c / 32; rows 4 w .. 4 w + 3 are bytes 4 (w % 4) ..
    // of half w / 4
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      // the top bytes of four signs, in k order; +-64 from their sign bits
      const uint32_t t01 = __builtin_amdgcn_perm(s[e][1], s[e][0], 0x0c0c0703u);
      const uint32_t t23 = __builtin_amdgcn_perm(s[e][3], s[e][2], 0x07030c0cu);
      const uint32_t bw = ((t01 | t23) & 0x80808080u) | 0x40404040u;
      const int c = 2 * lane + e;
      unsigned char *dst =
          smem + kBOff + b_bytes + (c >> 5) * kFragBytes + ((wave >> 2) * 32 + (c & 31)) * 16 + 4 * (wave & 3);
      *reinterpret_cast<uint32_t *>(dst) = bw;
    }
    ring_conv = (ring_conv + kRawBytes == kRingSlots * kRawBytes) ? 0 : ring_conv + kRawBytes;
  };

  // ---- activation wavefronts: copy c = v + 4 p of a k step is fragment (row fragment c / 3, digit c % 3)
  const __amdgpu_buffer_rsrc_t x_rsrc =
      rows_rsrc(a.xd, (uint32_t)(a.row_blocks * a.x_k_tiles * kDigits * kFragBytes));
  uint32_t x_off[kALoads]; // of the k step the next copy fetches
#pragma unroll
  for (int p = 0; p < kALoads; ++p) {
    const int c = v + 4 * p;
    int64_t rb = (int64_t)chunk * kRowFrags + c / kDigits;
    if (rb >= a.row_blocks)
      rb = a.row_blocks - 1; // (such rows are not multiplied)
    x_off[p] = __builtin_amdgcn_readfirstlane(
        (int)(((rb * a.x_k_tiles + t_begin) * kDigits + c % kDigits) * kFragBytes));
  }
  int a_left = T; // k steps not yet requested; past the last one the copy repeats it (uniform counters, valid addresses)
  auto issue_a = [&](int stage_bytes) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < kALoads; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void_t *)(smem + stage_bytes + (v + 4 * p) * kFragBytes), 16,
                                               lane * 16, x_off[p], 0, 0);
    if (--a_left > 0) {
#pragma unroll
      for (int p = 0; p < kALoads; ++p)
        x_off[p] += kDigits * kFragBytes;
    }
  };

  const bool idle = m0 + wave * 32 >= a.M; // no row of this wavefront exists
  auto multiply = [&](int stage_bytes, int b_bytes) __attribute__((always_inline)) {
    const uint4_t *sb = reinterpret_cast<const uint4_t *>(smem + kBOff + b_bytes) + lane;
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + stage_bytes + wave * kDigits * kFragBytes) + lane;
    i32x4_t av[kDigits];
#pragma unroll
    for (int d = 0; d < kDigits; ++d)
      av[d] = __builtin_bit_cast(i32x4_t, sa[d * 64]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const i32x4_t bv = __builtin_bit_cast(i32x4_t, sb[j * 64]);
#pragma unroll
      for (int d = 0; d < kDigits; ++d)
        acc[d][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[d], bv, acc[d][j], 0, 0, 0);
    }
  };

  // ---- prologue: k steps 0 and 1 of W landed, k step 0 converted; k step 0 of the digits landed
  if (weights) {
#pragma unroll
    for (int t = 0; t <= D; ++t)
      issue_w();
    NBLA_ROWS_WAIT_VMCNT(kWLoads * (D - 1)); // the first two of D + 1 groups of copies have landed
  } else {
    issue_a(0);
  }
  NBLA_ROWS_BARRIER();
  convert(0);
  if (!weights)
    NBLA_ROWS_WAIT_VMCNT(kConvStores); // all but the stores
  NBLA_ROWS_WAIT_LGKM0();
  NBLA_ROWS_BARRIER();

  // ---- main loop.  Iteration i multiplies k step i while every wavefront converts its rows of k step i + 1, whose
  // weights landed before the last barrier.  The weight wavefronts send the copy of k step i + 1 + D into the ring
  // slot k step i left and wait, before the barrier, for k step i + 2; the activation wavefronts request the digits
  // of k step i + 1 (into the stage k step i - 1 left) and wait for them before the barrier: they come out of the L2,
  // which every block of the XCD reads them from at about the same time.
  // Memory operations of a weight wavefront, in order: the D + 1 copy groups of the prologue (kWLoads each), the
  // kConvStores stores of a conversion, then per iteration one copy group and one conversion's stores.  Behind the
  // copies of k step i + 2 there are, at the wait, kWLoads (D - 2 - i) + kConvStores + (kWLoads + kConvStores) (i + 1)
  // operations while that k step comes from the prologue (i <= D - 2; the smallest of those counts, that of i = 0, is
  // used) and kConvStores + (kWLoads + kConvStores) (D - 1) after.  Of an activation wavefront: per iteration one copy
  // group and one conversion's stores; behind the copies of k step i + 1 there are those stores.
  // (The last iteration converts nothing, so its counts are short; nothing is read after it.)
  int a_cur = 0; // stage of k step i
  int b_cur = 0;
  for (int i = 0; i < T; ++i) {
    const int b_nxt = b_cur ^ kBTileBytes;
    // (the two wavefronts of a SIMD, w and w + 4, take conversion and multiplication in opposite orders; the
    // multiplication stands once in the code, so that the accumulators stay where they are)
    if (weights) {
      if (i + 1 < T)
        issue_w();
    } else {
      issue_a(a_cur ^ kAStageBytes);
      if (i + 1 < T)
        convert(b_nxt);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!idle)
      multiply(a_cur, b_cur);
    __builtin_amdgcn_sched_barrier(0);
    if (weights && i + 1 < T)
      convert(b_nxt);
    if (weights) {
      if (i <= D - 2)
        NBLA_ROWS_WAIT_VMCNT(kWLoads * (D - 2) + kConvStores + (kWLoads + kConvStores));
      else
        NBLA_ROWS_WAIT_VMCNT(kConvStores + (kWLoads + kConvStores) * (D - 1));
    } else {
      NBLA_ROWS_WAIT_VMCNT(kConvStores);
    }
    NBLA_ROWS_WAIT_LGKM0();
    NBLA_ROWS_BARRIER();
    a_cur ^= kAStageBytes;
    b_cur = b_nxt;
  }
  NBLA_ROWS_WAIT_VMCNT(0);
  NBLA_ROWS_BARRIER(); // every copy has landed: the stages may be overwritten

  // ---- epilogue.  Column sums of the eight wavefronts (rows 4 w .. 4 w + 3 of every k step), fixed order.
  float *red = reinterpret_cast<float *>(smem);
  *reinterpret_cast<float2_t *>(red + wave * kStripCols + 2 * lane) = colsum;
  if (a.zero_flag && col_ok && ((special >> lane) & 1))
    atomicOr(a.zero_flag, 1);
  __syncthreads();
  const int col_in_frag = lane & 31, row_half = lane >> 5;
  const bool sliced = a.slices > 1;
  float al[4], bi[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = 32 * j + col_in_frag;
    const int64_t n = n0 + c;
    const float cs = ((red[c] + red[kStripCols + c]) + (red[2 * kStripCols + c] + red[3 * kStripCols + c])) +
                     ((red[4 * kStripCols + c] + red[5 * kStripCols + c]) +
                      (red[6 * kStripCols + c] + red[7 * kStripCols + c]));
    al[j] = (a.alpha && !sliced) ? cs * a.inv_k : 1.0f;
    bi[j] = (a.bias && !sliced && n < a.N) ? a.bias[n] : -0.0f;
    if (chunk == 0 && wave == 0 && row_half == 0 && n < a.N) {
      if (sliced)
        a.partial[(int64_t)a.slices * a.M * a.N + (int64_t)slice * a.N + n] = cs;
      else if (a.alpha)
        a.alpha[n] = al[j];
    }
  }
  if (idle)
    return;
  float *out = sliced ? a.partial + (int64_t)slice * a.M * a.N : a.y;
#pragma unroll
  for (int rq = 0; rq < 4; ++rq) {
    const int64_t mq = m0 + wave * 32 + 4 * row_half + 8 * rq; // rows mq .. mq + 3
    if (mq >= a.M) // (the shifts are padded to whole row fragments, not beyond)
      continue;
    const i32x4_t sh = *reinterpret_cast<const i32x4_t *>(a.shift + mq);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int r = 4 * rq + e;
      const int shv = plain_shift(sh[e]);
      if (mq + e >= a.M || shv == kBadRow) // a row with a NaN or an infinity is the caller's
        continue;
      float *row = out + (mq + e) * a.N + n0 + col_in_frag;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // sum = d0 65536 + d1 256 + d2 exactly: high part u (|u| < 2^24), low part w in [0, 65536), one rounding
        const int d0 = acc[0][j][r] >> kSignScaleLog2, d1 = acc[1][j][r] >> kSignScaleLog2,
                  d2 = acc[2][j][r] >> kSignScaleLog2;
        int w = d1 * 256 + d2;
        const int u = d0 + (w >> 16);
        w &= 0xffff;
        float val = ldexpf(fmaf((float)u, 65536.0f, (float)w), -shv);
        val = val * al[j];
        val = val + bi[j];
        if (n0 + 32 * j + col_in_frag < a.N)
          __builtin_nontemporal_store(val, row + 32 * j);
      }
    }
  }
#endif
}

// y = (sum over the slices, in slice order) * alpha + bias with alpha = (sum of the slices' column sums) * (1 / K);
// a row marked kBadRow is left alone.  Thread = four columns of one row.
__global__ __launch_bounds__(256) void binary_affine_rows_finish(const float *__restrict__ partial,
                                                                 const int32_t *__restrict__ shift,
                                                                 float *__restrict__ alpha,
                                                                 const float *__restrict__ bias, float *__restrict__ y,
                                                                 int64_t M, int64_t N, int slices, float inv_k) {
  const int64_t n = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const int64_t m = blockIdx.y;
  if (n >= N)
    return;
  const float *cs = partial + (int64_t)slices * M * N + n;
  float4_t dot = *reinterpret_cast<const float4_t *>(partial + m * N + n);
  float4_t sum = *reinterpret_cast<const float4_t *>(cs);
  for (int s = 1; s < slices; ++s) {
    const float4_t d = *reinterpret_cast<const float4_t *>(partial + ((int64_t)s * M + m) * N + n);
    const float4_t c = *reinterpret_cast<const float4_t *>(cs + (int64_t)s * N);
    dot.x += d.x, dot.y += d.y, dot.z += d.z, dot.w += d.w;
    sum.x += c.x, sum.y += c.y, sum.z += c.z, sum.w += c.w;
  }
  if (alpha) {
    float4_t al;
    al.x = sum.x * inv_k, al.y = sum.y * inv_k, al.z = sum.z * inv_k, al.w = sum.w * inv_k;
    if (m == 0)
      *reinterpret_cast<float4_t *>(alpha + n) = al;
    dot.x = dot.x * al.x, dot.y = dot.y * al.y, dot.z = dot.z * al.z, dot.w = dot.w * al.w;
  }
  if (bias) {
    const float4_t b = *reinterpret_cast<const float4_t *>(bias + n);
    dot.x = dot.x + b.x, dot.y = dot.y + b.y, dot.z = dot.z + b.z, dot.w = dot.w + b.w;
  }
  if (plain_shift(shift[m]) != kBadRow)
    *reinterpret_cast<float4_t *>(y + m * N + n) = dot;
}

// Slices of K: as many as still give every block a CU of its own (blocks beyond the CUs would wait for a second
// round), at least sixteen k steps each.
int rows_slices(int64_t M, int64_t K, int64_t N) {
  const int64_t blocks = ceil_div(N, kStripCols) * ceil_div(M, kChunkRows);
  const int64_t by_cus = 256 / (blocks > 0 ? blocks : 1), by_k = ceil_div(K, kTileK) / 16;
  const int64_t s = by_cus < by_k ? by_cus : by_k;
  return s < 1 ? 1 : (s > 8 ? 8 : (int)s);
}

} // namespace

bool rows_affine_covers(const float *W, const float *Wb, const float *alpha, const float *bias, const float *y,
                        int64_t M, int64_t K, int64_t N) {
  // whole 16-byte runs of every row of W (and of y, alpha and bias for the launch that adds the slices); 32-bit byte
  // offsets inside W (the copies run kRingDepth k steps past the end); one chunk of the digit operand (int32 headroom)
  return M >= 1 && M <= kRowsMmaMaxRows && K >= 1 && Wb && N % 4 == 0 && aligned16(W) && aligned16(Wb) &&
         aligned16(alpha) && aligned16(bias) && aligned16(y) && K <= kChunkK &&
         (K + 32 * (kRingDepth + 2)) * N * 4 < (1ll << 31);
}

bool rows_affine_pays(int64_t M, int64_t K, int64_t N) {
  // Above the row counts the register-resident forms take, one chunk of rows, and enough blocks to occupy the CUs.
  // (With two chunks of rows both walk the strip and convert it, and a k step costs a block about a microsecond
  // whatever its rows: at K = 4096, N = 11008 the forward takes 76 / 79 / 88 us at M = 96 / 128 / 256 where the two
  // walks take 97 / 98 / 107, but 136 / 140 at M = 384 / 512 where they take 131 / 133.)
  return M > kFewRowsMaxRows && M <= kChunkRows &&
         ceil_div(N, kStripCols) * rows_slices(M, K, N) >= 128;
}

size_t rows_affine_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M < 1 || M > kRowsMmaMaxRows || K < 1 || N < 1)
    return 0;
  const int s = rows_slices(M, K, N);
  return s > 1 ? (size_t)s * (M + 1) * N * sizeof(float) : 0;
}

int launch_rows_affine(const void *xdigits, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                       int64_t M, int64_t K, int64_t N, float zero_to, int *zero_flag, void *workspace,
                       size_t workspace_bytes, hipStream_t stream) {
  const DigitOperand d = digit_operand(M, K);
  const char *base = static_cast<const char *>(xdigits);
  RowsArgs a;
  a.W = W;
  a.Wb = Wb;
  a.xd = reinterpret_cast<const uint4_t *>(base);
  a.shift = reinterpret_cast<const int32_t *>(base + d.shift_off);
  a.alpha = alpha;
  a.bias = bias;
  a.y = y;
  a.partial = static_cast<float *>(workspace);
  a.zero_flag = (zero_to == 1.0f || zero_to == -1.0f) ? nullptr : zero_flag;
  a.M = M, a.K = K, a.N = N;
  a.row_blocks = d.row_blocks;
  a.x_k_tiles = d.k_tiles;
  a.ksteps = (int)ceil_div(K, kTileK);
  a.strips = (int)ceil_div(N, kStripCols);
  a.chunks = (int)ceil_div(M, kChunkRows);
  a.slices = rows_slices(M, K, N);
  a.slice_steps = (int)ceil_div(a.ksteps, a.slices);
  a.slices = (int)ceil_div(a.ksteps, a.slice_steps); // no empty slice
  a.zero_to = zero_to;
  a.inv_k = (float)1 / K;
  if (a.slices > 1 && (workspace_bytes < (size_t)a.slices * (M + 1) * N * sizeof(float) || !aligned16(workspace)))
    return fail(NBLA_HIP_ERR_MEMORY, "one-walk binary affine workspace too small or misaligned.");
  static std::atomic<uint64_t> configured{0};
  const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(binary_affine_rows_kernel), kRowsLdsBytes, configured,
                                   "hipFuncSetAttribute(binary_affine_rows LDS size)");
  if (rc)
    return rc;
  const unsigned blocks = (unsigned)(ceil_div(a.strips, 8) * 8 * a.slices * a.chunks);
  hipLaunchKernelGGL(binary_affine_rows_kernel, dim3(blocks), dim3(kRowsThreads), kRowsLdsBytes, stream, a);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_rows");
  if (a.slices > 1) {
    hipLaunchKernelGGL(binary_affine_rows_finish, dim3((unsigned)ceil_div(N / 4, 256), (unsigned)M), dim3(256), 0,
                       stream, a.partial, a.shift, alpha, bias, y, M, N, a.slices, a.inv_k);
    NBLA_HIP_LAUNCH_CHECK("binary_affine_rows_finish");
  }
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
