// BinaryWeightAffine / BinaryConnectAffine forward for some hundreds of input rows (65 <= M <= 512), in ONE pass over
// W: the walk that writes Sign(W) and sums |W| per column also multiplies, on the int8 matrix cores.
//
// At these row counts the forward is still bound by the weights (4 B read and 4 B written per weight; the fp32 signs
// Wb are an output of the function), but the product is too large for one wavefront's registers.  The general path
// pays for that with two walks (binarise W to packed bits, then multiply them); here a block owns a 64-column strip
// of W over all of K and all rows of x:
//   * four "weight" wavefronts stream the strip through an LDS ring (global -> LDS copies, kRingDepth k steps of
//     32 rows ahead), turn every weight into its sign, store Wb, add |w| to their column sums and leave the signs in
//     LDS as the B fragments of v_mfma_i32_32x32x32_i8: byte 0x80 (-128) for a negative weight, 0 otherwise -- the
//     packed product's "column fragment 7" convention, so  sum_k q s = rowsum(q) + acc / 64  comes out of the same
//     exact integer epilogue (finish_dot);
//   * four "activation" wavefronts copy the k step's digit fragments of x (the operand split_digits_rows writes: three
//     balanced base-256 digits per value, one power-of-two scale per row) into a double-buffered LDS stage;
//   * all eight wavefronts multiply: wavefront w owns rows 64 w .. 64 w + 63 (32 w .. with at most 256 rows) of the
//     512 x 64 output tile, three int32 accumulator sets, 12 MFMAs per k step.
// The two roles keep separate memory counters: a wavefront's vmcnt retires in order, so a wavefront that waits for
// the digits it asked for one k step ago would also drain its weight copies, which must stay in flight for several
// k steps to cover HBM latency.  One workgroup barrier per k step hands the B tile and the digit stage over.
//
// Epilogue: the weight wavefronts' column sums are folded in a fixed order, alpha = colsum * ((float)1 / K)
// (binary_weight_affine.cpp:68), and  y = (rowsum + acc / 64) * 2^-shift * alpha + bias  in the order of operations of
// the packed product.  Rows of x that hold a NaN or an infinity are left to the caller (affine_redo_marked_rows).
// Sign(0) = quantize_zero_to other than +-1 cannot be a sign bit: the walk raises a flag when it meets such a weight
// and the caller's fp32 product (which runs only when the flag is up) replaces y.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kStripCols = 64;                    // columns of W per block: two column fragments
constexpr int kRowsThreads = 512;                 // eight wavefronts
constexpr int kRingDepth = 5;                     // k steps of W in flight ahead of the one being converted
constexpr int kRingSlots = kRingDepth + 1;
constexpr int kRawBytes = kTileK * kStripCols * 4; // one k step of the strip as fp32: 8 KiB
constexpr int kBTileBytes = 2 * kFragBytes;        // the signs of one k step: two column fragments
constexpr int kAStages = 2;
static_assert(10 * kRingDepth <= 63, "vmcnt is a 6-bit counter");

constexpr int rows_a_stage_bytes(int row_frags) { return row_frags * kDigits * kFragBytes; }
constexpr int rows_ring_off(int row_frags) { return kAStages * rows_a_stage_bytes(row_frags); }
constexpr int rows_b_off(int row_frags) { return rows_ring_off(row_frags) + kRingSlots * kRawBytes; }
constexpr int rows_lds_bytes(int row_frags) { return rows_b_off(row_frags) + 2 * kBTileBytes; }
static_assert(rows_lds_bytes(16) <= 160 * 1024, "the stages fit the CU's LDS");

struct RowsArgs {
  const float *W;
  float *Wb;
  const uint4_t *xd;     // digit fragments of x
  const long long *sums; // row sums of q
  const int32_t *shift;  // per-row scale exponents
  float *alpha;          // may be null (BinaryConnect)
  const float *bias;     // may be null
  float *y;
  int *zero_flag;        // raised when a weight is neither negative nor positive and zero_to is not +-1 (may be null)
  int64_t M, K, N;
  int64_t row_blocks, x_k_tiles;
  int ksteps;            // ceil(K / 32)
  float zero_to, inv_k;
};

// sign.hpp:48-50
__device__ __forceinline__ float rows_sign_of(float w, float zero_to, bool &plain) {
  const float one = __uint_as_float((__float_as_uint(w) & 0x80000000u) | 0x3f800000u);
  plain = __builtin_islessgreater(w, 0.0f);
  return plain ? one : zero_to;
}

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

// kRowFrags: row fragments (of 32 rows) of the block's tile, 16 or 8; a wavefront owns kRowFrags / 8 of them.
template <int kRowFrags>
__global__ __launch_bounds__(kRowsThreads, 1) void binary_affine_rows_kernel(RowsArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  typedef __attribute__((address_space(3))) void lds_void_t;
  constexpr int MF = kRowFrags / 8;
  constexpr int kAStage = rows_a_stage_bytes(kRowFrags);
  constexpr int kRingOff = rows_ring_off(kRowFrags), kBOff = rows_b_off(kRowFrags);
  constexpr int kALoads = kRowFrags * kDigits / 4; // fragment copies per activation wavefront and k step
  constexpr int D = kRingDepth;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool weights = wave >= 4; // role of this wavefront
  const int v = wave & 3;
  const int64_t n0 = (int64_t)blockIdx.x * kStripCols;
  const int T = a.ksteps;
  const uint32_t row_bytes = (uint32_t)(a.N * 4);
  const uint32_t step_bytes = row_bytes * kTileK;

  i32x16_t acc[kDigits][MF][2];
#pragma unroll
  for (int d = 0; d < kDigits; ++d)
#pragma unroll
    for (int f = 0; f < MF; ++f)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[d][f][j][r] = 0;

  // ---- weight wavefronts: the strip as a buffer that starts at its first column; reads past the end of W (k steps
  // beyond K, issued to keep the counters uniform) give zeros, stores past it are dropped
  const uint32_t strip_bytes = (uint32_t)((a.K * a.N - n0) * 4);
  const __amdgpu_buffer_rsrc_t w_rsrc = rows_rsrc(a.W + n0, strip_bytes);
  const __amdgpu_buffer_rsrc_t wb_rsrc = rows_rsrc(a.Wb + n0, strip_bytes);
  // copy: lane l fetches 16 bytes of row 8 v + l / 16 (+ 4 for the second copy) at columns 4 (l % 16) ..
  const uint32_t w_lane = (uint32_t)(8 * v + (lane >> 4)) * row_bytes + (uint32_t)(lane & 15) * 16u;
  // store: lane = column; columns past N go nowhere
  const uint32_t wb_lane = (n0 + lane < a.N) ? (uint32_t)(8 * v) * row_bytes + (uint32_t)lane * 4u : 0x80000000u;
  // (the k step's offset travels in the lane offsets, which the hardware range check covers for certain)
  uint32_t w_koff = 0;  // byte offset of the k step the next copy fetches
  uint32_t wb_koff = 0; // of the k step the next conversion stores
  int ring_next = 0;    // ring slot (bytes) of the next copy
  int ring_conv = 0;    // ring slot of the next conversion
  auto issue_w = [&]() __attribute__((always_inline)) {
    unsigned char *dst = smem + kRingOff + ring_next + v * 2048;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_void_t *)dst, 16, w_lane + w_koff, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_void_t *)(dst + 1024), 16, w_lane + w_koff + 4 * row_bytes, 0,
                                             0, 0);
    w_koff += step_bytes;
    ring_next = (ring_next + kRawBytes == kRingSlots * kRawBytes) ? 0 : ring_next + kRawBytes;
  };
  float colsum = 0.0f;
  bool all_plain = true;
  const bool col_ok = n0 + lane < a.N;
  int rows_left = (int)a.K - 8 * v; // rows of W from this wavefront's first row of the next conversion on
  // rows 8 v .. 8 v + 7 of the k step in ring slot ring_conv -> Wb, column sums, B tile `b_bytes`
  auto convert = [&](int b_bytes) __attribute__((always_inline)) {
    const float *raw = reinterpret_cast<const float *>(smem + kRingOff + ring_conv + v * 2048) + lane;
    float w[8], s[8];
#pragma unroll
    for (int r = 0; r < 8; ++r)
      w[r] = raw[r * kStripCols];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      bool plain;
      s[r] = rows_sign_of(w[r], a.zero_to, plain);
      all_plain = all_plain && (plain || !col_ok || r >= rows_left); // (what lies outside W reads as zero or garbage)
      colsum += fabsf(w[r]);
    }
    rows_left -= kTileK;
    uint32_t row_off = wb_lane + wb_koff;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(s[r]), wb_rsrc, row_off, 0, 2);
      row_off += row_bytes;
    }
    wb_koff += step_bytes;
    uint2_t bw;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // the top bytes of four signs, in k order
      const uint32_t t01 = __builtin_amdgcn_perm(__float_as_uint(s[4 * h + 1]), __float_as_uint(s[4 * h]), 0x0c0c0703u);
      const uint32_t t23 = __builtin_amdgcn_perm(__float_as_uint(s[4 * h + 3]), __float_as_uint(s[4 * h + 2]), 0x07030c0cu);
      bw[h] = (t01 | t23) & 0x80808080u;
    }
    unsigned char *dst = smem + kBOff + b_bytes + (lane >> 5) * kFragBytes + ((v >> 1) * 32 + (lane & 31)) * 16 + 8 * (v & 1);
    *reinterpret_cast<uint2_t *>(dst) = bw;
    ring_conv = (ring_conv + kRawBytes == kRingSlots * kRawBytes) ? 0 : ring_conv + kRawBytes;
  };

  // ---- activation wavefronts: copy c = v + 4 p of a k step is fragment (row fragment c / 3, digit c % 3)
  const __amdgpu_buffer_rsrc_t x_rsrc =
      rows_rsrc(a.xd, (uint32_t)(a.row_blocks * a.x_k_tiles * kDigits * kFragBytes));
  uint32_t x_soff[kALoads];
#pragma unroll
  for (int p = 0; p < kALoads; ++p) {
    const int c = v + 4 * p;
    int64_t rb = c / kDigits;
    if (rb >= a.row_blocks)
      rb = a.row_blocks - 1; // (such rows are not multiplied)
    x_soff[p] = __builtin_amdgcn_readfirstlane((int)((rb * a.x_k_tiles * kDigits + c % kDigits) * kFragBytes));
  }
  auto issue_a = [&](int stage_bytes) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < kALoads; ++p) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void_t *)(smem + stage_bytes + (v + 4 * p) * kFragBytes), 16,
                                               lane * 16, x_soff[p], 0, 0);
      x_soff[p] += kDigits * kFragBytes;
    }
  };

  const bool idle = (int64_t)wave * MF * 32 >= a.M; // no row of this wavefront exists
  auto multiply = [&](int stage_bytes, int b_bytes) __attribute__((always_inline)) {
    const uint4_t *sb = reinterpret_cast<const uint4_t *>(smem + kBOff + b_bytes) + lane;
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + stage_bytes + wave * MF * kDigits * kFragBytes) + lane;
    const i32x4_t b0 = __builtin_bit_cast(i32x4_t, sb[0]), b1 = __builtin_bit_cast(i32x4_t, sb[64]);
#pragma unroll
    for (int f = 0; f < MF; ++f)
#pragma unroll
      for (int d = 0; d < kDigits; ++d) {
        const i32x4_t av = __builtin_bit_cast(i32x4_t, sa[(f * kDigits + d) * 64]);
        acc[d][f][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b0, acc[d][f][0], 0, 0, 0);
        acc[d][f][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b1, acc[d][f][1], 0, 0, 0);
      }
  };

  // ---- prologue: k step 0 converted and staged
  if (weights) {
#pragma unroll
    for (int t = 0; t <= D; ++t)
      issue_w();
    NBLA_ROWS_WAIT_VMCNT(2 * D); // the first of D + 1 pairs has landed
    convert(0);
  } else {
    issue_a(0);
    NBLA_ROWS_WAIT_VMCNT(0);
  }
  NBLA_ROWS_WAIT_LGKM0();
  NBLA_ROWS_BARRIER();

  // ---- main loop.  Iteration i multiplies k step i while k step i + 1 is converted (weight wavefronts; the copy of
  // k step i + 1 + D goes into the ring slot k step i left) and its digits are copied (activation wavefronts).
  // Memory operations of a weight wavefront, in order: the D + 1 copy pairs of the prologue, eight stores, then per
  // iteration one copy pair and eight stores.  Behind the copies of k step i + 1 there are, at the wait, 2 D + 8 + 8 i
  // operations while that k step comes from the prologue (i < D; the smallest of those counts is used) and 10 D after.
  int a_cur = 0, b_cur = 0;
  for (int i = 0; i < T; ++i) {
    const int a_nxt = a_cur ^ kAStage, b_nxt = b_cur ^ kBTileBytes;
    if (i + 1 < T) {
      if (weights) {
        issue_w();
        if (i < D)
          NBLA_ROWS_WAIT_VMCNT(2 * D + 8);
        else
          NBLA_ROWS_WAIT_VMCNT(10 * D);
        convert(b_nxt);
      } else {
        issue_a(a_nxt);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!idle)
      multiply(a_cur, b_cur);
    __builtin_amdgcn_sched_barrier(0);
    if (!weights)
      NBLA_ROWS_WAIT_VMCNT(0);
    NBLA_ROWS_WAIT_LGKM0();
    NBLA_ROWS_BARRIER();
    a_cur = a_nxt;
    b_cur = b_nxt;
  }
  NBLA_ROWS_WAIT_VMCNT(0);

  // ---- epilogue.  Column sums of the four weight wavefronts (rows 8 v .. 8 v + 7 of every k step), fixed order.
  float *red = reinterpret_cast<float *>(smem);
  if (weights) {
    red[v * kStripCols + lane] = colsum;
    if (a.zero_flag && !all_plain)
      atomicOr(a.zero_flag, 1);
  }
  __syncthreads();
  const int col_in_frag = lane & 31, row_half = lane >> 5;
  float al[2], bi[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int c = 32 * j + col_in_frag;
    const int64_t n = n0 + c;
    const float cs = (red[c] + red[kStripCols + c]) + (red[2 * kStripCols + c] + red[3 * kStripCols + c]);
    al[j] = a.alpha ? cs * a.inv_k : 1.0f;
    bi[j] = (a.bias && n < a.N) ? a.bias[n] : -0.0f;
    if (a.alpha && wave == 0 && row_half == 0 && n < a.N)
      a.alpha[n] = al[j];
  }
  if (idle)
    return;
  // accumulators hold -128 x (sum of the digits under negative weights): the packed product's column fragment 7
  const int c_hi = 2, c_mid = 512, c_lo = 2;
#pragma unroll
  for (int f = 0; f < MF; ++f) {
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const int64_t mq = ((int64_t)wave * MF + f) * 32 + 4 * row_half + 8 * rq; // rows mq .. mq + 3
      if (mq >= a.M) // (the metadata arrays are padded to whole row fragments, not beyond)
        continue;
      const i32x4_t sum01 = *reinterpret_cast<const i32x4_t *>(a.sums + mq);
      const i32x4_t sum23 = *reinterpret_cast<const i32x4_t *>(a.sums + mq + 2);
      const i32x4_t sh = *reinterpret_cast<const i32x4_t *>(a.shift + mq);
      const uint32_t lo_w[4] = {(uint32_t)sum01.x, (uint32_t)sum01.z, (uint32_t)sum23.x, (uint32_t)sum23.z};
      const int hi_w[4] = {sum01.y, sum01.w, sum23.y, sum23.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * rq + e;
        const int shv = plain_shift(sh[e]);
        if (mq + e >= a.M || shv == kBadRow) // a row with a NaN or an infinity is the caller's
          continue;
        const int s_hi = (int)((lo_w[e] >> 16) | ((uint32_t)hi_w[e] << 16)), s_lo = (int)(lo_w[e] & 0xffffu);
        float *row = a.y + (mq + e) * a.N + n0 + col_in_frag;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int m0 = acc[0][f][j][r] >> 7, m1 = acc[1][f][j][r] >> 7, m2 = acc[2][f][j][r] >> 7;
          int u = __mul24(m0, c_hi) + s_hi;
          int w = __mul24(m1, c_mid) + (__mul24(m2, c_lo) + s_lo);
          u += w >> 16;
          w &= 0xffff;
          float val = ldexpf(fmaf((float)u, 65536.0f, (float)w), -shv);
          val = val * al[j];
          val = val + bi[j];
          if (n0 + 32 * j + col_in_frag < a.N)
            __builtin_nontemporal_store(val, row + 32 * j);
        }
      }
    }
  }
#endif
}

template <int kRowFrags> int launch_rows(const RowsArgs &a, hipStream_t stream) {
  auto kernel = binary_affine_rows_kernel<kRowFrags>;
  constexpr int kSmem = rows_lds_bytes(kRowFrags);
  static std::atomic<uint64_t> configured{0};
  const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), kSmem, configured,
                                   "hipFuncSetAttribute(binary_affine_rows LDS size)");
  if (rc)
    return rc;
  hipLaunchKernelGGL(kernel, dim3((unsigned)ceil_div(a.N, kStripCols)), dim3(kRowsThreads), kSmem, stream, a);
  NBLA_HIP_LAUNCH_CHECK("binary_affine_rows");
  return NBLA_HIP_OK;
}

} // namespace

bool rows_affine_covers(const float *W, const float *Wb, int64_t M, int64_t K, int64_t N) {
  // whole 16-byte runs of every row of W; 32-bit byte offsets inside W (the copies run kRingDepth k steps past the
  // end); one chunk of the digit operand (int32 headroom)
  return M >= 1 && M <= kRowsMmaMaxRows && K >= 1 && Wb && N % 4 == 0 && aligned16(W) && aligned16(Wb) &&
         K <= kChunkK && (K + 32 * (kRingDepth + 2)) * N * 4 < (1ll << 31);
}

bool rows_affine_pays(int64_t M, int64_t N) {
  // above the row counts the register-resident forms take, and with enough strips to occupy the CUs
  return M > kFewRowsMaxRows && ceil_div(N, kStripCols) >= 128;
}

int launch_rows_affine(const void *xdigits, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                       int64_t M, int64_t K, int64_t N, float zero_to, int *zero_flag, hipStream_t stream) {
  const DigitOperand d = digit_operand(M, K);
  const char *base = static_cast<const char *>(xdigits);
  RowsArgs a;
  a.W = W;
  a.Wb = Wb;
  a.xd = reinterpret_cast<const uint4_t *>(base);
  a.sums = reinterpret_cast<const long long *>(base + d.sum_off);
  a.shift = reinterpret_cast<const int32_t *>(base + d.shift_off);
  a.alpha = alpha;
  a.bias = bias;
  a.y = y;
  a.zero_flag = (zero_to == 1.0f || zero_to == -1.0f) ? nullptr : zero_flag;
  a.M = M, a.K = K, a.N = N;
  a.row_blocks = d.row_blocks;
  a.x_k_tiles = d.k_tiles;
  a.ksteps = (int)ceil_div(K, kTileK);
  a.zero_to = zero_to;
  a.inv_k = (float)1 / K;
  if (M <= 256)
    return launch_rows<8>(a, stream);
  return launch_rows<16>(a, stream);
}

} // namespace nbla_hip
