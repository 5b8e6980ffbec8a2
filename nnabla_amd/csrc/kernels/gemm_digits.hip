// Product of two real-valued matrices on the int8 matrix cores: y[m, n] = sum_k A[m, k] * B[n, k] with both
// operands as digit operands (per row a power-of-two scale and three balanced base-256 int8 digits, see
// gemm_layout.hpp).  With qa = a0 * 2^16 + a1 * 2^8 + a2 and qb likewise,
//     qa * qb = a0 b0 * 2^32 + (a0 b1 + a1 b0) * 2^24 + (a0 b2 + a1 b1 + a2 b0) * 2^16 + (lower terms)
// and the six leading digit products are accumulated exactly in three int32 accumulators per output (one per power
// of 256); the dropped terms are below 2^-23 of |row max| * |column max| per k.  The epilogue combines the three
// sums in integer arithmetic, converts once and applies the two scales, so the result does not depend on the order
// of summation.  Used for the weight gradients (x^T . dy), where neither factor is a sign matrix.
//
// Tiling: 128 x 128 outputs per block of four wavefronts (2 x 2, 64 x 64 each: 2 x 2 fragments x 3 accumulators =
// 192 registers), k in tiles of 32 (one v_mfma_i32_32x32x32_i8 fragment).
#include "common.hpp"
#include "copy_pipeline.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

#include <type_traits>

namespace nbla_hip {
namespace {

typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct GemmDigitsArgs {
  const uint4_t *ad, *bd; // [row blocks][k tiles][3][64] uint4 each
  const int32_t *ashift, *bshift, *bshift_narrow, *bflag;
  const float *bias;
  float *y;
  int64_t M, N, a_row_blocks, b_row_blocks, k_tiles, step_begin, step_end, blocks_m, blocks_n;
  int64_t inner, outer_stride, n_stride;
  int accumulate; // add to y instead of overwriting it
  int finish;     // last chunk of the contraction: add the bias
  // contraction split over blockIdx.y (outputs of few tiles): split z multiplies the k tiles
  // [step_begin + z * split_tiles, + split_tiles) and writes its own dense [M, N] partial result at y + z * M * N
  int64_t split_tiles; // 0: no split
};

constexpr int kBM = 128, kBN = 128, kThreads = 256, kWaves = 4;
constexpr int kSegs = 4;               // 32-row fragments per tile side
constexpr int kSegVec = kDigits * 64;  // uint4 per fragment and k step
constexpr int kSideVec = kSegs * kSegVec;
constexpr int kStageBytes = 2 * kSideVec * 16; // 24 KiB: the A and B fragments of one k tile
constexpr int kChunks = 2 * kSegs * kDigits;   // 1 KiB copies per k tile
constexpr int kPerWave = kChunks / kWaves;     // 6
// Three LDS stages when two blocks share a CU; six (the whole LDS) when the output has so few tiles that a CU holds
// one block anyway: with one wavefront per SIMD a k tile is multiplied in a few hundred cycles and the copies need
// the longer head start to cover the memory latency.
constexpr int kStagesShared = 3, kStagesAlone = 6;

// Which of a wavefront's kPerWave copy slots a call of copy_next issues (the list of a k tile is ordered so that
// every form of the product needs a prefix of each wavefront's share), and how many that makes: the unit in which the
// loop's wait counts copies in flight.
constexpr bool copy_slot_used(int p, bool one_a, bool narrow, int groups) {
  const int all_waves = kWaves * groups, per_tile = kChunks / all_waves;
  return one_a ? p < (2 * kSegs / all_waves) * groups
               : !(narrow && p % per_tile >= (kSegs * kDigits + kSegs) / all_waves);
}
constexpr int copies_per_call(bool one_a, bool narrow, int groups) {
  int n = 0;
  for (int p = 0; p < kPerWave; ++p)
    n += copy_slot_used(p, one_a, narrow, groups) ? 1 : 0;
  return n;
}

// Workgroup barrier without the memory fence of __syncthreads() (which would wait for every global -> LDS copy in
// flight, including those of later k tiles); the waits that matter are explicit.
#define NBLA_BARRIER()                                                                                                 \
  do {                                                                                                                 \
    asm volatile("" ::: "memory");                                                                                     \
    __builtin_amdgcn_s_barrier();                                                                                      \
    asm volatile("" ::: "memory");                                                                                     \
  } while (0)
// vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
#define NBLA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8))

// Staging: global -> LDS copies bypass the registers (one wavefront instruction moves one 1 KiB fragment); kStages
// LDS buffers hold consecutive k tiles and the copy of tile t + kStages - 1 is issued while tile t is multiplied.  Two blocks
// share a CU (256 registers per lane: 192 accumulators + the 12 operand quads of a tile), so one block's LDS reads
// and barrier waits are covered by the other's MFMAs.
// kNarrow: the B operand holds every value in its lowest digit alone (a small integer): three products
// a_t x b2 -> accumulator t, nothing dropped, and only the lowest-digit fragments of B are copied.
// kTopB (a form of kNarrow): every row of the tile's B row blocks is a one-digit row of a row-scaled operand (its value
// sits in the top digit: power-of-two weights once INQ has fixed them): the same three products with b0 in place of
// b2, and the factor 2^16 of the top digit in the epilogue.
// kOneA (only with kNarrow): every row of the tile's A row blocks is a one-digit row (gemm_layout.hpp: its value sits
// in the top digit): a single product a0 x b2 -> accumulator 0, and only the top-digit fragments of A and the
// lowest-digit fragments of B are copied (eight per k tile, dealt evenly over the wavefronts).  Same bits as the other
// forms: the other digits are zero.
// kGroups = 2 (outputs of at most one tile per CU): eight wavefronts, two groups of four; group g multiplies the k
// tiles g, g + 2, ... of the same output tile (a stage then holds two consecutive k tiles), so every SIMD has a second
// wavefront to issue from while the first waits.  At the end the groups swap halves of their int32 accumulators
// through LDS (exactly) and group g finishes row fragment g of each wavefront tile.
template <bool kNarrow, bool kOneA, int kStages, int kGroups, bool kTopB = false>
__device__ __forceinline__ void gemm_digits_tile(const GemmDigitsArgs &a, unsigned char *smem) {
#if defined(__HIP_DEVICE_COMPILE__) // the host pass only needs the launch stub; the body uses LDS address-space pointers
  static_assert(kGroups == 1 || kGroups == 2, "k groups per block");
  static_assert(!kOneA || kNarrow, "the one-digit A form is implemented for one-digit B operands");
  static_assert(!kTopB || kNarrow, "the top-digit B form is a narrow form");
  constexpr int kBDigit = kTopB ? 0 : kDigits - 1; // the one digit of B a narrow form multiplies
  constexpr int kAllWaves = kWaves * kGroups;
  constexpr int kGroupStageBytes = kGroups * kStageBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int group = wave_all / kWaves, wave = wave_all % kWaves;
  const int wm = wave & 1, wn = wave >> 1;
  int64_t bm, bn;
  band_tile<8>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn); // two blocks per CU: 64 resident tiles per XCD = 8 x 8

  // This wavefront's copies.  The 24 fragments of a k tile are numbered u: [0, 12) the A fragments (row block,
  // digit), [12, 16) the lowest-digit B fragments, [16, 24) the other B fragments; wavefront w takes
  // u = q * kAllWaves + w, so each takes the same number (two thirds of its list) of the sixteen that the narrow form
  // needs.  Copy p of a wavefront is fragment q = p % kPerTile of k tile p / kPerTile of the stage.
  constexpr int kPerTile = kChunks / kAllWaves; // 6 or 3
  // kOneA: the eight fragments f of a k tile that hold anything ([0, 4) A top digit, [4, 8) B lowest digit);
  // wavefront w takes f = q * kAllWaves + w
  constexpr int kOnePerTile = 2 * kSegs / kAllWaves; // 2 or 1
  const uint4_t *cur[kPerWave], *cur_last[kPerWave];
  int dest[kPerWave]; // byte offset inside a stage
#pragma unroll
  for (int p = 0; p < kPerWave; ++p) {
    int sub, side, seg, d;
    if (kOneA) {
      sub = p / kOnePerTile;
      const int f = (p - sub * kOnePerTile) * kAllWaves + wave_all;
      side = f / kSegs, seg = f % kSegs, d = side ? kBDigit : 0;
      if (p >= kOnePerTile * kGroups)
        sub = 0, side = 0, seg = 0; // unused slot
    } else {
      sub = p / kPerTile;
      const int q = p - sub * kPerTile;
      const int u = q * kAllWaves + wave_all;
      if (u < kSegs * kDigits)
        side = 0, seg = u / kDigits, d = u - seg * kDigits;
      else if (u < kSegs * kDigits + kSegs)
        side = 1, seg = u - kSegs * kDigits, d = kBDigit;
      else // the two digits of B that a narrow form leaves out
        side = 1, seg = (u - kSegs * kDigits - kSegs) / (kDigits - 1),
        d = (u - kSegs * kDigits - kSegs) % (kDigits - 1) + (kTopB ? 1 : 0);
    }
    dest[p] = sub * kStageBytes + ((side * kSegs + seg) * kDigits + d) * kFragBytes;
    int64_t rb = (side ? bn : bm) * kSegs + seg;
    const int64_t limit = side ? a.b_row_blocks : a.a_row_blocks;
    if (rb >= limit)
      rb = limit - 1; // clamped: those rows / columns are not stored
    const uint4_t *base = (side ? a.bd : a.ad) + (rb * a.k_tiles * kDigits + d) * 64;
    cur[p] = base + (a.step_begin + sub) * kSegVec;
    cur_last[p] = base + (a.step_end - kGroups + sub) * kSegVec;
  }
  typedef __attribute__((address_space(3))) void lds_void_t;
  // narrow: the first two thirds of each k tile's list (A fragments and lowest-digit B fragments)
  constexpr int kNeeded = (kSegs * kDigits + kSegs) / kAllWaves; // 4 or 2 per k tile
  constexpr int kCopies = kOneA ? kOnePerTile * kGroups : (kNarrow ? kNeeded * kGroups : kPerWave);
  auto copy_next = [&](int buf) {
#pragma unroll
    for (int p = 0; p < kPerWave; ++p) {
      if (!copy_slot_used(p, kOneA, kNarrow, kGroups))
        continue;
      __builtin_amdgcn_global_load_lds(cur[p] + lane, (lds_void_t *)(smem + buf * kGroupStageBytes + dest[p]), 16, 0,
                                       0);
      const uint4_t *next = cur[p] + kGroups * kSegVec;
      cur[p] = next < cur_last[p] ? next : cur_last[p]; // the last calls copy the final tile again
    }
  };

  i32x16_t acc[2][2][3];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[i][j][t][r] = 0;

  // The number of most recently issued k tiles the wait at the top of a tile may leave in flight, from the model of
  // this loop's order of copies, waits, barriers and LDS reads (copy_pipeline.hpp)
  constexpr int kLoopWait = pipeline::one_tile_loop_wait(kStages, kStages - 1);
  static_assert(kLoopWait >= 0 && pipeline::one_tile_safe(kStages, kStages - 1, kLoopWait),
                "the copy pipeline hands a buffer over too early");
  static_assert(pipeline::counter_fits(kLoopWait, kPerWave), "vmcnt is a 6-bit counter");
  static_assert(copies_per_call(kOneA, kNarrow, kGroups) == kCopies, "the wait counts the copies a call issues");
#pragma unroll
  for (int d = 0; d < kStages - 1; ++d)
    copy_next(d);
  int buf = 0;
  for (int64_t kt = a.step_begin; kt < a.step_end; kt += kGroups) {
    // tile kt has landed (the copies of the kStages - 2 tiles after it may still be in flight) and every wavefront
    // is done with the buffer tile kt - 1 occupied, which tile kt + kStages - 1 takes over
    NBLA_WAIT_VMCNT(kLoopWait * kCopies);
    NBLA_BARRIER();
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + buf * kGroupStageBytes + group * kStageBytes);
    const uint4_t *sb = sa + kSideVec;
    i32x4_t af[2][3], bf[2][3];
    // digit by digit: the first products need the top digits' four fragments only
    if (kNarrow) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
        bf[i][kBDigit] = __builtin_bit_cast(i32x4_t, sb[((wn * 2 + i) * kDigits + kBDigit) * 64 + lane]);
    }
#pragma unroll
    for (int d = 0; d < 3; ++d)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (!kOneA || d == 0)
          af[i][d] = __builtin_bit_cast(i32x4_t, sa[((wm * 2 + i) * kDigits + d) * 64 + lane]);
        if (!kNarrow)
          bf[i][d] = __builtin_bit_cast(i32x4_t, sb[((wn * 2 + i) * kDigits + d) * 64 + lane]);
      }
    copy_next(buf == 0 ? kStages - 1 : buf - 1);
    // Issue order (sched_group_barrier: 0x100 = LDS read, 0x008 = MFMA, 0x020 = the copies' loads): the fragments of
    // the first products, then one further read per MFMA, then one copy per MFMA, instead of twelve reads and the
    // copies in a row before the first MFMA -- a wavefront cannot feed the matrix pipe while it issues a batch of other
    // instructions (the weight-gradient product of 4096 x 4096 x 11008: 1.14 -> 1.08 ms).
    constexpr int kFirstReads = kOneA ? 4 : (kNarrow ? 4 : 4);
    constexpr int kAllReads = kOneA ? 4 : (kNarrow ? 8 : 12);
    constexpr int kAllMfmas = kOneA ? 4 : (kNarrow ? 12 : 24);
    static_assert(kAllReads - kFirstReads + kCopies <= kAllMfmas, "more reads and copies than MFMAs to deal them out to");
    if (kOneA) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i][0], bf[j][kBDigit], acc[i][j][0], 0, 0, 0);
    } else if (kNarrow) {
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i][t], bf[j][kBDigit], acc[i][j][t], 0, 0, 0);
    } else {
      // digit pairs (a digit, b digit) -> accumulator a + b
      constexpr int da[6] = {0, 0, 1, 0, 1, 2};
      constexpr int db[6] = {0, 1, 0, 2, 1, 0};
#pragma unroll
      for (int t = 0; t < 6; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j][da[t] + db[t]] =
                __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i][da[t]], bf[j][db[t]], acc[i][j][da[t] + db[t]], 0, 0, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, kFirstReads, 0);
#pragma unroll
    for (int q = 0; q < kAllReads - kFirstReads; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int q = 0; q < kCopies; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAllMfmas - (kAllReads - kFirstReads) - kCopies, 0);
    __builtin_amdgcn_sched_barrier(0);
    buf = (buf + 1 == kStages) ? 0 : buf + 1;
  }
  NBLA_WAIT_VMCNT(0);

  if (kGroups == 2) {
    // swap: every wavefront hands the row fragment it does not finish to its partner in the other group, one
    // accumulator set at a time (8 wavefronts x 2 fragments x 16 registers x 64 lanes x 4 B = 64 KiB per round)
    int *xs = reinterpret_cast<int *>(smem);
    const int partner = wave_all ^ kWaves;
#pragma unroll
    for (int t = 0; t < (kOneA ? 1 : 3); ++t) {
      __syncthreads(); // the stages (first round) or the previous round's values have been read
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (i != group) {
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              xs[((wave_all * 2 + j) * 16 + r) * 64 + lane] = acc[i][j][t][r];
        }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (i == group) {
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              acc[i][j][t][r] += xs[((partner * 2 + j) * 16 + r) * 64 + lane];
        }
    }
  }

  // y = (acc0 * 2^16 + acc1 * 2^8 + acc2) * 2^(16 - sa - sb); the narrow form has no factor 2^16 (b is its low digit)
  // unless b is the top digit of a row-scaled operand.
  // Row by row: the row's offset (one 32-bit division when m is folded into two output indices) and shift are
  // formed once and serve both column fragments.
  const int col_in_frag = lane & 31, row_half = lane >> 5;
  const int32_t *bshift = (kNarrow && !kTopB) ? a.bshift_narrow : a.bshift;
  int64_t n_col[2];
  int32_t sb_n[2];
  float bias_n[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    n_col[j] = bn * kBN + (wn * 2 + j) * 32 + col_in_frag;
    const bool in = n_col[j] < a.N;
    sb_n[j] = in ? plain_shift(bshift[n_col[j]]) : 0; // one-digit rows store their shift with a bias
    bias_n[j] = (in && a.bias && a.finish) ? a.bias[n_col[j]] : 0.0f;
  }
  const bool add_bias = a.bias && a.finish;
  const uint32_t inner = (uint32_t)a.inner;
  // the 32 row shifts of each row fragment: one coalesced load up front (lane l holds row l % 32), handed out by
  // shuffles, instead of a dependent global load per row inside the store loop
  int32_t row_shift[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int64_t m = bm * kBM + (wm * 2 + i) * 32 + (lane & 31);
    const int64_t last = a.a_row_blocks * kFragRows - 1;
    row_shift[i] = plain_shift(a.ashift[m < last ? m : last]);
  }
  // Two copies of the stores, with and without reading y back first: with that load anywhere in the loop the
  // compiler waits for all outstanding memory operations before every output, and the stores before it are
  // outstanding memory operations -- each store would wait for the previous one.
  auto store_rows = [&](auto accumulate_c) __attribute__((always_inline)) {
    constexpr bool kAcc = decltype(accumulate_c)::value;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (kGroups == 2 && i != group)
        continue;
      const int64_t m0 = bm * kBM + (wm * 2 + i) * 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * row_half + (r & 3);
        const int32_t sa_m = __shfl(row_shift[i], row);
        const int64_t m = m0 + row;
        if (m >= a.M)
          continue;
        int64_t off;
        if (inner == 1u) {
          off = m * a.outer_stride;
        } else {
          const uint32_t mu = (uint32_t)m, q = mu / inner; // m < 2^31: operand rows are counted in 32 bits
          off = (int64_t)q * a.outer_stride + (mu - q * inner);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (n_col[j] >= a.N)
            continue;
          float v;
          if (sa_m == kBadRow || sb_n[j] == kBadRow) {
            v = __uint_as_float(0x7fc00000u);
          } else {
            // t = acc0 * 2^16 + acc1 * 2^8 + acc2 regrouped as hi * 2^16 + lo with 0 <= lo < 2^17 and |hi| < 2^30 (32-bit
            // integer steps only), then one fused multiply-add: exact while |hi| < 2^24, else rounded twice (2^-24 of t)
            const int a0 = acc[i][j][0][r], a1 = acc[i][j][1][r], a2 = acc[i][j][2][r];
            const int hi = a0 + (a1 >> 8) + (a2 >> 16);
            const int lo = ((a1 & 0xff) << 8) + (a2 & 0xffff);
            const float t = fmaf((float)hi, 65536.0f, (float)lo);
            // the two shifts are applied one after the other: each stays inside ldexpf's exponent range
            v = ldexpf(ldexpf(t, ((kNarrow && !kTopB) ? 0 : 16) - sa_m), -sb_n[j]);
          }
          float *dst = a.y + off + n_col[j] * a.n_stride;
          if (kAcc)
            v = *dst + v;
          if (add_bias)
            v = v + bias_n[j];
          *dst = v;
        }
      }
    }
  };
  if (a.accumulate)
    store_rows(std::true_type());
  else
    store_rows(std::false_type());
#endif
}

template <int kStages, int kGroups>
__global__ __launch_bounds__(kThreads * kGroups, kGroups == 1 ? 2 : 1) void gemm_digits_kernel(GemmDigitsArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  if (a.split_tiles > 0) {
    const int64_t begin = a.step_begin + (int64_t)blockIdx.y * a.split_tiles;
    a.step_end = begin + a.split_tiles < a.step_end ? begin + a.split_tiles : a.step_end;
    a.step_begin = begin;
    a.y += (int64_t)blockIdx.y * a.M * a.N;
  }
  if (*a.bflag == 0) { // uniform over the grid
    // are all rows of this tile's A row blocks one-digit rows?  (rows past the operand clamp to its last row)
    int64_t bm, bn;
    band_tile<8>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn);
    const int64_t rows = a.a_row_blocks * kFragRows;
    bool one = true;
    for (int r = threadIdx.x; r < kBM; r += kThreads * kGroups) {
      const int64_t m = bm * kBM + r;
      one = one && one_digit_row(a.ashift[m < rows ? m : rows - 1]);
    }
    if (__syncthreads_and(one))
      gemm_digits_tile<true, true, kStages, kGroups>(a, smem);
    else
      gemm_digits_tile<true, false, kStages, kGroups>(a, smem);
  } else {
    // all rows of this tile's B row blocks one-digit rows (of a row-scaled operand; column-scaled ones never are)?
    int64_t bm, bn;
    band_tile<8>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn);
    const int64_t arows = a.a_row_blocks * kFragRows, brows = a.b_row_blocks * kFragRows;
    bool one_b = true, one_a = true;
    for (int r = threadIdx.x; r < kBN; r += kThreads * kGroups) {
      const int64_t n = bn * kBN + r;
      one_b = one_b && one_digit_row(a.bshift[n < brows ? n : brows - 1]);
    }
    for (int r = threadIdx.x; r < kBM; r += kThreads * kGroups) {
      const int64_t m = bm * kBM + r;
      one_a = one_a && one_digit_row(a.ashift[m < arows ? m : arows - 1]);
    }
    one_b = __syncthreads_and(one_b);
    one_a = __syncthreads_and(one_a);
    if (one_b && one_a)
      gemm_digits_tile<true, true, kStages, kGroups, true>(a, smem);
    else if (one_b)
      gemm_digits_tile<true, false, kStages, kGroups, true>(a, smem);
    else
      gemm_digits_tile<false, false, kStages, kGroups>(a, smem);
  }
}

// y (+)= sum over the splits of their partial results, in split order, then the bias: what the single-launch epilogue
// does with one value.
__global__ __launch_bounds__(256) void gemm_digits_split_sum(const float *__restrict__ partial, int splits, int64_t M,
                                                             int64_t N, float *__restrict__ y, int64_t inner,
                                                             int64_t outer_stride, int64_t n_stride,
                                                             const float *__restrict__ bias, int accumulate) {
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / N, n = i - m * N;
    float v = partial[i];
    for (int z = 1; z < splits; ++z)
      v += partial[(int64_t)z * total + i];
    const int64_t q = m / inner;
    float *dst = y + q * outer_stride + (m - q * inner) + n * n_stride;
    if (accumulate)
      v = *dst + v;
    if (bias)
      v = v + bias[n];
    *dst = v;
  }
}

// The same for outputs whose consecutive elements in memory are consecutive rows m (n_stride != 1: convolution
// results [sample, channel, position]): a 32 x 32 tile is read along n and, through LDS, written along m.
__global__ __launch_bounds__(256) void gemm_digits_split_sum_rows(const float *__restrict__ partial, int splits,
                                                                  int64_t M, int64_t N, float *__restrict__ y,
                                                                  int64_t inner, int64_t outer_stride, int64_t n_stride,
                                                                  const float *__restrict__ bias, int accumulate) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // ty: 0..7
  const int64_t n0 = (int64_t)blockIdx.x * 32, m0 = (int64_t)blockIdx.y * 32, total = M * N;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty + 8 * i, n = n0 + tx;
    float v = 0.0f;
    if (m < M && n < N) {
      v = partial[m * N + n];
      for (int z = 1; z < splits; ++z)
        v += partial[(int64_t)z * total + m * N + n];
    }
    tile[ty + 8 * i][tx] = v;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + tx, n = n0 + ty + 8 * i;
    if (m < M && n < N) {
      float v = tile[tx][ty + 8 * i];
      const int64_t q = m / inner;
      float *dst = y + q * outer_stride + (m - q * inner) + n * n_stride;
      if (accumulate)
        v = *dst + v;
      if (bias)
        v = v + bias[n];
      *dst = v;
    }
  }
}

// Splits of the contraction for an output of `tiles` 128 x 128 tiles and `k_tiles` k tiles: as many as fill the CUs
// with one block each, at least 16 k tiles per split; 1 = no split.
inline int64_t digit_product_splits(int64_t tiles, int64_t k_tiles) {
  if (tiles * 2 > 256 || k_tiles < 32)
    return 1;
  const int64_t by_cus = 256 / tiles, by_k = k_tiles / 16;
  return by_cus < by_k ? by_cus : by_k;
}

} // namespace

size_t gemm_digits_split_bytes(int64_t M, int64_t K, int64_t N) {
  const int64_t k_tiles = digit_k_tiles(K) < kChunkK / kTileK ? digit_k_tiles(K) : kChunkK / kTileK;
  const int64_t s = digit_product_splits(ceil_div(M, kBM) * ceil_div(N, kBN), k_tiles);
  return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

int launch_gemm_digits(const void *adigits, const void *bdigits, const float *bias, float *y, int64_t M, int64_t K,
                       int64_t N, int64_t inner, int64_t outer_stride, int64_t n_stride, hipStream_t stream,
                       bool accumulate, void *split_ws, size_t split_ws_bytes) {
  if (M >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "digit product: more than 2^31 - 1 rows or columns.");
  const DigitOperand da = digit_operand(M, K), db = digit_operand(N, K);
  static std::atomic<uint64_t> configured[3];
  int rc = allow_dynamic_lds(reinterpret_cast<const void *>(gemm_digits_kernel<kStagesShared, 1>),
                             kStagesShared * kStageBytes, configured[0], "hipFuncSetAttribute(gemm_digits LDS size)");
  if (!rc)
    rc = allow_dynamic_lds(reinterpret_cast<const void *>(gemm_digits_kernel<kStagesAlone, 1>),
                           kStagesAlone * kStageBytes, configured[1], "hipFuncSetAttribute(gemm_digits LDS size)");
  if (!rc)
    rc = allow_dynamic_lds(reinterpret_cast<const void *>(gemm_digits_kernel<kStagesShared, 2>),
                           kStagesShared * 2 * kStageBytes, configured[2], "hipFuncSetAttribute(gemm_digits LDS size)");
  if (rc)
    return rc;
  GemmDigitsArgs a;
  a.ad = static_cast<const uint4_t *>(adigits);
  a.bd = static_cast<const uint4_t *>(bdigits);
  a.ashift = reinterpret_cast<const int32_t *>(static_cast<const char *>(adigits) + da.shift_off);
  a.bshift = reinterpret_cast<const int32_t *>(static_cast<const char *>(bdigits) + db.shift_off);
  a.bshift_narrow = reinterpret_cast<const int32_t *>(static_cast<const char *>(bdigits) + db.sum_off);
  a.bflag = reinterpret_cast<const int32_t *>(static_cast<const char *>(bdigits) + db.flag_off);
  a.bias = bias;
  a.y = y;
  a.M = M;
  a.N = N;
  a.a_row_blocks = da.row_blocks;
  a.b_row_blocks = db.row_blocks;
  a.k_tiles = da.k_tiles;
  a.blocks_m = ceil_div(M, kBM);
  a.blocks_n = ceil_div(N, kBN);
  a.inner = inner;
  a.outer_stride = outer_stride;
  a.n_stride = n_stride;
  // chunks of kChunkK contraction elements keep the int32 sums below 2^31; their fp32 results are added up
  const int64_t tiles_per_chunk = kChunkK / kTileK;
  for (int64_t t0 = 0, chunk = 0; t0 < a.k_tiles; t0 += tiles_per_chunk, ++chunk) {
    a.step_begin = t0;
    a.step_end = (t0 + tiles_per_chunk < a.k_tiles) ? t0 + tiles_per_chunk : a.k_tiles;
    a.accumulate = (accumulate || chunk > 0) ? 1 : 0;
    a.finish = a.step_end == a.k_tiles ? 1 : 0;
    a.split_tiles = 0;
    const unsigned blocks = (unsigned)(a.blocks_m * a.blocks_n);
    const int64_t chunk_tiles = a.step_end - a.step_begin;
    int64_t splits = split_ws ? digit_product_splits(blocks, chunk_tiles) : 1;
    while (splits > 1 && (size_t)splits * M * N * sizeof(float) > split_ws_bytes)
      --splits;
    if (splits > 1) {
      // few output tiles, long contraction: every split writes a dense partial result, summed in split order
      GemmDigitsArgs part = a;
      part.split_tiles = ceil_div(ceil_div(chunk_tiles, splits), 8) * 8;
      splits = ceil_div(chunk_tiles, part.split_tiles);
      part.y = static_cast<float *>(split_ws);
      part.inner = 1, part.outer_stride = N, part.n_stride = 1;
      part.accumulate = 0, part.bias = nullptr;
      hipLaunchKernelGGL((gemm_digits_kernel<kStagesShared, 2>), dim3(blocks, (unsigned)splits), dim3(2 * kThreads),
                         kStagesShared * 2 * kStageBytes, stream, part);
      NBLA_HIP_LAUNCH_CHECK("gemm_digits");
      if (n_stride != 1 && ceil_div(M, 32) <= 65535) {
        hipLaunchKernelGGL(gemm_digits_split_sum_rows, dim3((unsigned)ceil_div(N, 32), (unsigned)ceil_div(M, 32)),
                           dim3(256), 0, stream, static_cast<const float *>(split_ws), (int)splits, M, N, y, inner,
                           outer_stride, n_stride, a.finish ? bias : nullptr, a.accumulate);
      } else {
        int64_t sum_blocks = ceil_div(M * N, 256);
        if (sum_blocks > 4096)
          sum_blocks = 4096;
        hipLaunchKernelGGL(gemm_digits_split_sum, dim3((unsigned)sum_blocks), dim3(256), 0, stream,
                           static_cast<const float *>(split_ws), (int)splits, M, N, y, inner, outer_stride, n_stride,
                           a.finish ? bias : nullptr, a.accumulate);
      }
      NBLA_HIP_LAUNCH_CHECK("gemm_digits_split_sum");
      continue;
    }
    if (blocks <= 256 && chunk_tiles % 2 == 0) // at most one block per CU: eight wavefronts, two k groups (k tiles
                                               // come in multiples of 8)
      hipLaunchKernelGGL((gemm_digits_kernel<kStagesShared, 2>), dim3(blocks), dim3(2 * kThreads),
                         kStagesShared * 2 * kStageBytes, stream, a);
    else if (blocks <= 384) // fewer than 1.5 blocks per CU
      hipLaunchKernelGGL((gemm_digits_kernel<kStagesAlone, 1>), dim3(blocks), dim3(kThreads),
                         kStagesAlone * kStageBytes, stream, a);
    else
      hipLaunchKernelGGL((gemm_digits_kernel<kStagesShared, 1>), dim3(blocks), dim3(kThreads),
                         kStagesShared * kStageBytes, stream, a);
    NBLA_HIP_LAUNCH_CHECK("gemm_digits");
  }
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
