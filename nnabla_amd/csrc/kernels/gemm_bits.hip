// y = (x . B) * alpha + bias for sign-binarised weights B, on the gfx950 matrix cores' int8 path.
//
// x arrives as the digit operand: per row a power-of-two scale and, per element, the integer q = rint(x * 2^s) as
// three balanced base-256 digits (int8).  B arrives as one bit per weight and is expanded in registers (one AND per
// register) to bytes b * 2^F, F the column fragment's index inside its 256-column group.  v_mfma_i32_32x32x32_i8 accumulates  sum_k digit * b  exactly in int32, one accumulator per digit, and
// the epilogue divides the 2^F out and forms  rowsum(q) - 2 * (acc0 * 65536 + acc1 * 256 + acc2)  =  sum_k q * (+-1)  in integer arithmetic
// before the single conversion to fp32.  The result is therefore independent of tiling and summation order, and its
// only error is the rounding of x to 24 significant bits relative to the largest magnitude of its row.
//
// Work decomposition: a block of kWavesM x kWavesN wavefronts owns a BM x BN output tile and walks K in steps of
// 64 (two k tiles).  Per step it stages
//   X: BM/32 row blocks x (2 k tiles x 3 digits) fragments = BM/32 * 6 KiB
//   B: 2 k tiles x BN/64 column groups x 64 packed words   = BN * 8 B
// from HBM/L2 straight into LDS (several steps ahead, one barrier per step).  X fragments are read back with one
// conflict-free 128-bit LDS load per lane; four packed words become the four registers of any of eight column fragments
// with one AND each.
// Every wavefront keeps 3 x MF x NF accumulator tiles, so blocks are sized for one wavefront per SIMD.
#include "common.hpp"
#include "conv_geom.hpp"
#include "copy_pipeline.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

#include <hip/hip_ext.h>
#include <type_traits>
#include <utility>
#include <vector>

namespace nbla_hip {
namespace {

typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct GemmBitsArgs {
  const uint4_t *xd;      // digit fragments
  const long long *sums;  // row sums of this k chunk
  const int32_t *shift;   // per-row scale exponents
  const uint32_t *bits;   // packed weights
  const float *alpha;     // may be null
  const float *bias;      // may be null
  float *y;
  int64_t M, N;
  int64_t n_begin, n_end; // column range this launch produces (n_begin a multiple of 256)
  int64_t row_blocks;     // of the digit operand
  int64_t x_k_tiles;      // k tiles of the digit operand (even)
  int64_t wide_groups;    // 256-column groups of the packed operand
  int64_t step_begin, step_end; // k steps (of two k tiles) this launch covers
  int64_t blocks_m, blocks_n;
  int64_t inner, outer_stride, n_stride; // output addressing
  int accumulate; // add to y instead of overwriting it (k chunks after the first)
  int finish;     // apply alpha and bias (last k chunk)
  // contraction split over blockIdx.y (outputs of very few tiles): split z multiplies the k steps
  // [step_begin + z * split_steps, + split_steps) and writes a dense [M, N] partial result at y + z * M * N; only
  // split 0 adds the row sums
  int64_t split_steps; // 0: no split
  int use_sums;
  int keep_bad_rows; // rows marked kBadRow are left as they are in y (the caller has computed them) instead of NaN
  // unfolding product (gemm_bits_unfold_kernel): the rows are the unfolded windows of x, converted to digits in the
  // kernel; xd, sums and shift are unused
  const float *ux;
  ConvGeom ug;
  int64_t ugrp;
  const int *skip_if; // non-zero word: the launch does nothing (may be null)
  int32_t *shift_out; // unfolding product only (may be null): the rows' scale exponents, kBadRow for a window holding
                      // a NaN or an infinity, written for the caller that recomputes such windows
};

// LDS buffers (stages resident) per tile shape: what fits the block's share of the CU's 160 KiB, at most six.
constexpr int gemm_bits_stage_bytes(int BM, int BN, int waves_k) {
  return ((BM / 32) * 2 * kDigits * kFragBytes + 2 * BN * 4) * waves_k;
}
constexpr int gemm_bits_stages(int BM, int BN, int waves_mn, int waves_k) {
  const int stage = gemm_bits_stage_bytes(BM, BN, waves_k);
  const int budget = (waves_mn * waves_k >= 8 ? 144 : 72) * 1024; // two blocks per CU below eight wavefronts
  return budget / stage >= 6 ? 6 : (budget / stage >= 3 ? budget / stage : 3);
}
// LDS bytes of a block: the stages, or the accumulator exchange of the k groups if that is larger
constexpr int gemm_bits_lds_bytes(int BM, int BN, int waves_m, int waves_n, int waves_k) {
  const int stages = gemm_bits_stages(BM, BN, waves_m * waves_n, waves_k) * gemm_bits_stage_bytes(BM, BN, waves_k);
  const int exchange = (waves_k - 1) * (BM / 32) * (BN / 32) * 4096; // one digit: 32x32 int32 per fragment
  return stages > exchange ? stages : exchange;
}

// Past the stages (and the exchange area) the LDS holds what the epilogue needs besides the accumulators: the block's
// row sums (int64) and shifts, and its columns' alpha and bias.  They are loaded while the first copies are in flight
// and read back from LDS at the end, so the epilogue starts without a round trip to memory.
constexpr int gemm_bits_epilogue_bytes(int BM, int BN) { return (BM * 12 + BN * 8 + 255) / 256 * 256; }

// sum_k q_k * (+-1) as fp32 from the three digit accumulators and the row sum (hi * 65536 + lo), scaled by 2^-shift.
// Integer arithmetic up to the last step: the high and low parts are combined by one fused multiply-add, whose
// operands are exact (|hi part| < 2^24, low part reduced to 16 bits).
//
// The accumulators of column fragment `frag` carry the factor 2^frag (-128 for frag 7: 0x80 as int8); without it a
// digit sum m_d is below 2^21 in magnitude (at most kChunkK products of magnitude 128), so the sign of the factor and
// the weights -2, -512, -2 of  rowsum - 2 (m_0 65536 + m_1 256 + m_2)  go into 24-bit multiply-adds.
// A row that holds a non-finite value gets hi_scale = NaN instead of 65536 (its digits are all zero): NaN comes out.
struct FragScale {
  int shift;             // frag
  int c_hi, c_mid, c_lo; // -2, -512, -2, negated for frag 7
};
__device__ __forceinline__ FragScale frag_scale(int frag) {
  const int sgn = frag == 7 ? -1 : 1;
  FragScale f{frag, -2 * sgn, -512 * sgn, -2 * sgn};
  // kept in scalar registers as values the compiler does not see through: a known multiplier makes it expand the
  // 24-bit multiply-add into shifts with a sign extension of the other factor, three instructions for one
  asm volatile("" : "+s"(f.c_hi), "+s"(f.c_mid), "+s"(f.c_lo));
  return f;
}
__device__ __forceinline__ float finish_dot(int a0, int a1, int a2, int s_hi, int s_lo, int neg_shift, float hi_scale,
                                            const FragScale &f) {
  const int m0 = a0 >> f.shift, m1 = a1 >> f.shift, m2 = a2 >> f.shift;
  int u = __mul24(m0, f.c_hi) + s_hi;
  int v = __mul24(m1, f.c_mid) + (__mul24(m2, f.c_lo) + s_lo);
  u += v >> 16;
  v &= 0xffff;
  const float r = fmaf((float)u, hi_scale, (float)v);
  return ldexpf(r, neg_shift);
}
// per row: the exponent and the high part's scale
__device__ __forceinline__ int row_neg_shift(int shift) { return shift == kBadRow ? 0 : -shift; }
__device__ __forceinline__ float row_hi_scale(int shift) { return shift == kBadRow ? __builtin_nanf("") : 65536.0f; }

// Workgroup barrier without the memory fence of __syncthreads(): the fence would wait for every outstanding
// global -> LDS copy, including those issued for later k steps.  The waits that matter are explicit (wait_copies);
// the empty asm statements keep the compiler from moving LDS accesses across the barrier.
#define NBLA_BARRIER()                                                                                                 \
  do {                                                                                                                 \
    asm volatile("" ::: "memory");                                                                                     \
    __builtin_amdgcn_s_barrier();                                                                                      \
    asm volatile("" ::: "memory");                                                                                     \
  } while (0)

// vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
#define NBLA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8))

// kSwap exchanges the MFMA operand roles (the instruction computes the transposed 32x32 tile), which puts
// consecutive m on consecutive lanes of the accumulator: the store pattern for outputs whose m index is contiguous.
//
// Staging: global -> LDS copies bypass the registers (global_load_lds): one wavefront instruction moves one 1 KiB
// digit fragment, or 64 packed words, to the same lane order in LDS.  kStages LDS buffers hold consecutive k steps;
// the copy of step ks + kStages - 1 is issued while step ks is being multiplied.
//
// kWavesK > 1 splits the contraction inside the block: wavefront group wk multiplies k steps wk, wk + kWavesK, ...
// of the same output tile (a stage then holds kWavesK consecutive k steps) and the groups' int32 accumulators are
// added through LDS at the end, exactly.  Used when the output has too few tiles to occupy the CUs.
//
// kUsed = 1: every row of the block's row blocks is a one-digit row (gemm_layout.hpp: the two lower digits are zero).
// Only the top-digit fragments are copied and multiplied, into the top accumulator; the lower accumulators stay
// zero and the epilogue is the same.  A third of the MFMAs and a third of the digit traffic, same bits.
// The unfolding product keeps two buffers of kUnfoldSteps stages of the plain kernel each; past them (and past the
// k groups' exchange area, which reuses the buffers at the end) the LDS holds the row sums, row maxima and row shifts,
// then the table of decoded unfolded columns (16 bytes each).
constexpr int kUnfoldSteps = 2;
constexpr int kUnfoldRowTaps = 65; // a row's byte offsets of its taps (64 at most) and one entry that is never valid
// sums, maxima, shifts; the taps' table; alpha, bias; the rows' tap offsets
constexpr int kUnfoldMetaBytes = 512 + 64 * 16 + 2 * 256 * 4 + 32 * kUnfoldRowTaps * 4;
constexpr uint32_t kUnfoldNowhere = 0x80000000u; // a byte offset past every input the fused product accepts
constexpr int unfold_meta_off(int BM, int BN, int waves_m, int waves_n, int waves_k) {
  const int stages = 2 * kUnfoldSteps * gemm_bits_stage_bytes(BM, BN, waves_k);
  const int exchange = (waves_k - 1) * (BM / 32) * (BN / 32) * 4096;
  return stages > exchange ? stages : exchange;
}

// Main loop of the unfolding product: the block's 32 rows are unfolded windows of x (rows m = (sample, output
// position), columns kk = (channel, kernel tap), as im2col lays them out) that are never written to memory.  The block
//  1. decodes the taps (at most 64) into {offset, displacements} and every column kk into an LDS table {byte offset of
//     its channel's plane, 4 x its tap} (kk >= Kg: the tap entry that is never valid);
//  2. finds for each row which taps fall inside the input and the row's largest magnitude, and from that the row's
//     power-of-two scale, exactly as the stand-alone unfold kernels do; then writes, per row and tap, the byte offset
//     of that tap's element of channel 0 in x, or an offset past the end of x when the tap falls outside the input
//     (or the row holds a non-finite value, or lies past the last row).  An element of the unfolded matrix is then
//     one bounds-checked buffer load at (row's tap offset + column's channel offset): out of range reads give 0,
//     so the loop has no validity tests and no selects;
//  3. walks the contraction in stages of eight k tiles with two LDS buffers.  Wavefront w produces k tile w of a
//     stage: lane l gathers the sixteen values of row l % 32, k slots (l / 32) * 16 + 0..15, turns them into digits,
//     writes them where the fragment's lane l holds them and adds their sum to the row's sum; it also moves the
//     packed words of the tile to LDS.  Everything is loaded into registers two stages ahead (the loads of stage s+2
//     are in flight while stage s is multiplied and stage s+1 converted and stored), one barrier per stage.  (Plain
//     loads, not global -> LDS copies: with such a copy outstanding the compiler makes every LDS read wait for all
//     loads, the gathered ones included.)
// `multiply(buffer offset)` runs the wavefront's MFMAs of one stage of the plain kernel (kWavesK k steps).
template <int BM, int BN, int kWavesM, int kWavesN, int kWavesK, int kStageBytes, int kStepBytes, int kABytes,
          class Multiply>
__device__ __forceinline__ void unfold_main_loop(const GemmBitsArgs &a, unsigned char *smem, int64_t bm, int64_t bn,
                                                 int wave, int lane, bool idle, Multiply multiply) {
  static_assert(BM == 32 && BN == kWideGroup && kWavesM * kWavesN * kWavesK == 8 && kWavesK == 2 && kUnfoldSteps == 2,
                "thread mapping of the unfolding product: eight wavefronts, eight k tiles per stage");
  constexpr int kThreads = 512, kStageTiles = 2 * kWavesK * kUnfoldSteps, kStageK = kStageTiles * kTileK;
  constexpr int kBufBytes = kUnfoldSteps * kStageBytes;
  constexpr int kMetaOff = unfold_meta_off(BM, BN, kWavesM, kWavesN, kWavesK);
  typedef __attribute__((address_space(3))) void lds_void_t;
  const ConvGeom &g = a.ug;
  long long *s_sums = reinterpret_cast<long long *>(smem + kMetaOff);
  uint32_t *s_amax = reinterpret_cast<uint32_t *>(smem + kMetaOff + 256);
  int32_t *s_shift = reinterpret_cast<int32_t *>(smem + kMetaOff + 384);
  typedef int i32x2_t __attribute__((ext_vector_type(2)));
  i32x2_t *table = reinterpret_cast<i32x2_t *>(smem + kMetaOff + kUnfoldMetaBytes);
  uint32_t *row_taps = reinterpret_cast<uint32_t *>(smem + kMetaOff + 512 + 64 * 16 + 2 * 256 * 4);
  float *s_alpha = reinterpret_cast<float *>(smem + kMetaOff + 512 + 64 * 16), *s_bias = s_alpha + 256;
  const int tid = threadIdx.x;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size;
  const int k_tiles = (int)a.x_k_tiles, nstages = k_tiles / kStageTiles;
  // scratch of step 2, in the space of the stage buffers (unused until step 3): per-pixel channel maxima of the
  // input positions the block's windows touch, and the runs of consecutive rows that lie in one sample ("segments")
  constexpr int kPixCap = 4096, kPixPerLane = 8; // pixels in all segments / 64-pixel rounds of one segment
  static_assert(kPixCap * 4 + 4 * 32 * 4 + 4 <= kMetaOff, "the scratch of step 2 fits the stage buffers");
  uint32_t *s_pix = reinterpret_cast<uint32_t *>(smem);
  int *seg_lo = reinterpret_cast<int *>(smem + kPixCap * 4), *seg_hi = seg_lo + 32, *seg_n = seg_lo + 64;
  int *row_seg = seg_lo + 96, *seg_count = seg_lo + 128;

  // 1. the decoded taps, then the columns (one division per column: channel = column / taps)
  i32x4_t *taps_table = reinterpret_cast<i32x4_t *>(smem + kMetaOff + 512);
  const int taps = (int)g.k_size;
  if (tid < taps) {
    const int K1 = g.k[1], K2 = g.k[2];
    int q = tid;
    const int k2 = q % K2;
    q /= K2;
    const int k1 = q % K1, k0 = q / K1;
    const int e0 = k0 * g.dil[0], e1 = k1 * g.dil[1], e2 = k2 * g.dil[2];
    i32x4_t t;
    t.x = (e0 * in1 + e1) * in2 + e2;
    t.y = e0 | (e1 << 16);
    t.z = e2;
    t.w = 0;
    taps_table[tid] = t;
  }
  {
    for (int kk = tid; kk < k_tiles * kTileK; kk += kThreads) {
      const int c = kk / taps, tap = kk - c * taps;
      i32x2_t e;
      e.x = kk < (int)g.Kg ? c * plane * 4 : 0;
      e.y = kk < (int)g.Kg ? tap * 4 : (kUnfoldRowTaps - 1) * 4;
      table[kk] = e;
    }
    if (tid < 32) {
      s_amax[tid] = 0u;
      s_sums[tid] = 0;
      seg_lo[tid] = 0x7fffffff;
      seg_hi[tid] = -1;
    }
    for (int i = tid; i < kPixCap; i += kThreads)
      s_pix[i] = 0u;
    if (tid < 256) { // the block's columns' alpha and bias: the epilogue reads them from LDS
      const int64_t col = a.n_begin + bn * BN + tid;
      const int64_t nc = col < a.N ? col : a.N - 1;
      s_alpha[tid] = (a.finish && a.alpha) ? a.alpha[nc] : 1.0f;
      s_bias[tid] = (a.finish && a.bias) ? a.bias[nc] : -0.0f;
    }
  }
  // this thread's row (the same for both of its roles: lane % 32)
  const int r = lane & 31, half = lane >> 5;
  const int64_t m = bm * BM + r;
  const bool in_range = m < a.M;
  const int64_t n = in_range ? m / g.out_sp_size : 0;
  int p = in_range ? (int)(m - n * g.out_sp_size) : 0;
  const int o2 = p % g.out_sp[2];
  p /= g.out_sp[2];
  const int o1 = p % g.out_sp[1];
  const int o0 = p / g.out_sp[1];
  const int b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
  const int origin = (b0 * in1 + b1) * in2 + b2; // may be negative; only added to the offsets of taps inside the input
  const float *xn = a.ux + (n * g.C + a.ugrp * g.Cg) * g.in_sp_size;
  __syncthreads();

  // 2. the row's taps inside the input (a 64-bit mask), and its largest magnitude.  The rows of a block are
  // consecutive output positions, so their windows overlap: instead of gathering every row's window (taps x channels
  // loads per row, a few values per cache line), the block first takes the maximum over the channels of every input
  // position its windows can touch -- per segment one run [lo, hi] of the flattened plane, read with consecutive
  // lanes on consecutive positions -- and a row's maximum is then the maximum of its taps' positions.
  if (tid < 32) {
    // segments: wavefront 0, lanes 0..31 hold rows 0..31
    const unsigned long long starts = __ballot(in_range && (r == 0 || m / g.out_sp_size != (m - 1) / g.out_sp_size));
    const int seg = __popcll(starts & ((2ull << r) - 1ull)) - 1;
    row_seg[r] = in_range ? seg : 0;
    if (in_range) {
      int last = 0; // the largest tap offset
      for (int t = 0; t < taps; ++t)
        last = max(last, taps_table[t].x);
      const int lo = origin > 0 ? origin : 0, hi = origin + last < plane - 1 ? origin + last : plane - 1;
      atomicMin(&seg_lo[seg], lo);
      atomicMax(&seg_hi[seg], hi);
      seg_n[seg] = (int)n;
    }
    if (r == 0)
      *seg_count = __popcll(starts & 0xffffffffull);
  }
  __syncthreads();
  uint32_t mask_lo = 0u, mask_hi = 0u;
  const int nseg = *seg_count;
  // blocks whose positions do not fit the scratch take the gathering form
  bool by_pixels = true;
  int my_base = 0, total = 0;
  for (int sgm = 0; sgm < (by_pixels ? nseg : 0); ++sgm) {
    const int len = seg_hi[sgm] - seg_lo[sgm] + 1;
    if (sgm == row_seg[r])
      my_base = total;
    total += len > 0 ? len : 0;
    by_pixels = by_pixels && len <= 64 * kPixPerLane;
  }
  by_pixels = by_pixels && total <= kPixCap;
  if (by_pixels) {
    const int Cg = (int)g.Cg;
    int base = 0;
    for (int sgm = 0; sgm < nseg; ++sgm) {
      const int lo = seg_lo[sgm], len = seg_hi[sgm] - lo + 1;
      if (len <= 0)
        continue;
      const float *xs = a.ux + ((int64_t)seg_n[sgm] * g.C + a.ugrp * g.Cg) * g.in_sp_size + lo;
      for (int p0 = 0; p0 < len; p0 += 64) {
        const int pix = p0 + lane;
        const bool live = pix < len;
        const float *src = xs + (live ? pix : 0);
        uint32_t amax = 0u;
        // channels wave, wave + 8, ...: sixteen loads in flight
        for (int c0 = wave; c0 < Cg; c0 += 8 * 16) {
          float v[16];
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const int c = c0 + 8 * j;
            v[j] = src[(int64_t)(c < Cg ? c : wave) * plane];
          }
#pragma unroll
          for (int j = 0; j < 16; ++j)
            if (c0 + 8 * j < Cg)
              amax = max(amax, __float_as_uint(v[j]) & 0x7fffffffu);
        }
        if (live && amax)
          atomicMax(&s_pix[base + pix], amax);
      }
      base += len;
    }
    __syncthreads();
    uint32_t amax = 0u;
    const int rel = my_base + origin - seg_lo[row_seg[r]];
    for (int t = 0; t < taps; ++t) {
      const i32x4_t e = taps_table[t];
      const int i0 = b0 + (e.y & 0xffff), i1 = b1 + (int)((uint32_t)e.y >> 16), i2 = b2 + e.z;
      const bool ok = in_range && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                      (unsigned)i2 < (unsigned)in2;
      if (ok) {
        if (t < 32)
          mask_lo |= 1u << t;
        else
          mask_hi |= 1u << (t - 32);
        amax = max(amax, s_pix[rel + e.x]);
      }
    }
    if (tid < 32)
      s_amax[r] = amax;
  } else {
    {
      uint32_t amax = 0u;
      const int slice = wave * 2 + half, Cg = (int)g.Cg;
      // (tap, round of 256 channels) pairs, the loads of one pair in flight while the previous one is reduced
      const int rounds = (Cg + 255) / 256, pairs = taps * rounds;
      float v[2][16];
      bool okv[2];
      int c0v[2];
      auto issue = [&](int pair, int slot) __attribute__((always_inline)) {
        const int t = pair / rounds, c0 = slice + (pair - t * rounds) * 256;
        const i32x4_t e = taps_table[t];
        const int i0 = b0 + (e.y & 0xffff), i1 = b1 + (int)((uint32_t)e.y >> 16), i2 = b2 + e.z;
        const bool ok = in_range && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                        (unsigned)i2 < (unsigned)in2;
        if (ok) {
          if (t < 32)
            mask_lo |= 1u << t;
          else
            mask_hi |= 1u << (t - 32);
        }
        const float *src = xn + (ok ? origin + e.x : 0);
  #pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int c = c0 + 16 * j;
          v[slot][j] = src[(int64_t)(c < Cg ? c : slice) * plane];
        }
        okv[slot] = ok;
        c0v[slot] = c0;
      };
      auto reduce = [&](int slot) __attribute__((always_inline)) {
  #pragma unroll
        for (int j = 0; j < 16; ++j)
          if (okv[slot] && c0v[slot] + 16 * j < Cg)
            amax = max(amax, __float_as_uint(v[slot][j]) & 0x7fffffffu);
      };
      issue(0, 0);
      for (int pair = 0; pair < pairs; pair += 2) {
        if (pair + 1 < pairs)
          issue(pair + 1, 1);
        reduce(0);
        if (pair + 2 < pairs)
          issue(pair + 2, 0);
        if (pair + 1 < pairs)
          reduce(1);
      }
      if (amax)
        atomicMax(&s_amax[r], amax);
    }
  }
  __syncthreads();
  if (tid < 32) {
    const uint32_t amax = s_amax[tid];
    int s = 0;
    if (amax >= 0x7f800000u) {
      s = kBadRow;
    } else if (amax != 0u) {
      s = 22 - binade_exponent(binade_of(amax));
      if (rintf(ldexpf(__uint_as_float(amax), s)) > (float)kDigitMax)
        --s;
    }
    s_shift[tid] = s;
    if (a.shift_out && bn == 0 && in_range)
      a.shift_out[m] = s;
    // the row's taps as byte offsets into x; a row holding a NaN or an infinity is not read (its outputs become NaN
    // in the epilogue), nor is a tap outside the input
    const uint32_t first = (uint32_t)(((n * g.C + a.ugrp * g.Cg) * g.in_sp_size + origin) * 4);
    for (int t = 0; t < taps; ++t) {
      const bool ok = s != kBadRow && (((t < 32 ? mask_lo >> t : mask_hi >> (t - 32)) & 1u) != 0u);
      row_taps[tid * kUnfoldRowTaps + t] = ok ? first + (uint32_t)taps_table[t].x * 4u : kUnfoldNowhere;
    }
    row_taps[tid * kUnfoldRowTaps + kUnfoldRowTaps - 1] = kUnfoldNowhere;
  }
  __syncthreads();

  // 3. the stages
  const int s_row = s_shift[r];
  // x as a buffer: reads at offsets past its end (kUnfoldNowhere + any channel offset) return zero
  const uint64_t xbase = reinterpret_cast<uint64_t>(a.ux);
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<void *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(xbase >> 32)) << 32) |
                               (uint32_t)__builtin_amdgcn_readfirstlane((int)xbase)),
      0, __builtin_amdgcn_readfirstlane((int)(g.outer * g.C * g.in_sp_size * 4)), 0x00020000);
  const uint32_t *my_taps = row_taps + r * kUnfoldRowTaps;
  // k tile `wave` of a stage sits in stage wave / 4 of the buffer, k step (wave % 4) / 2, tile wave % 2 of the step
  const int tile_off = (wave >> 2) * kStageBytes + ((wave & 3) >> 1) * kStepBytes;
  int64_t wg = a.n_begin / kWideGroup + bn;
  if (wg >= a.wide_groups)
    wg = a.wide_groups - 1;
  const uint4_t *words_src = reinterpret_cast<const uint4_t *>(a.bits) + wg * 64 + lane;
  auto gather = [&](int stage, float (&v)[16], uint4_t &words) __attribute__((always_inline)) {
    words = words_src[(int64_t)(stage * kStageTiles + wave) * a.wide_groups * 64];
    const int kb = stage * kStageK + wave * kTileK + half * 16;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const i32x2_t e = table[kb + j];
      const uint32_t at = my_taps[e.y >> 2] + (uint32_t)e.x;
      v[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(xrsrc, (int)at, 0, 0));
    }
  };
  auto emit = [&](int stage, const float (&v)[16], const uint4_t &words) __attribute__((always_inline)) {
    uint32_t w[3][4];
    int qv[16], part = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      qv[j] = (int)rintf(ldexpf(v[j], s_row)); // masked values are 0.0f -> 0 whatever the shift
      part += qv[j];
    }
    pack_digits(qv, w);
    uint4_t *dst = reinterpret_cast<uint4_t *>(smem + (stage & 1) * kBufBytes + tile_off +
                                               (wave & 1) * kDigits * kFragBytes) + lane;
#pragma unroll
    for (int d = 0; d < kDigits; ++d) {
      uint4_t o;
      o.x = w[d][0], o.y = w[d][1], o.z = w[d][2], o.w = w[d][3];
      dst[d * 64] = o;
    }
    *(reinterpret_cast<uint4_t *>(smem + (stage & 1) * kBufBytes + tile_off + kABytes + (wave & 1) * kFragBytes) +
      lane) = words;
    if (part != 0)
      atomicAdd(reinterpret_cast<unsigned long long *>(&s_sums[r]), (unsigned long long)(long long)part);
  };
  // one stage: `ahead` receives the loads of stage s+2, `next` holds those of stage s+1
  auto stage_step = [&](int s, float (&ahead)[16], uint4_t &words_ahead, const float (&next)[16],
                        const uint4_t &words_next) __attribute__((always_inline)) {
    if (s + 2 < nstages)
      gather(s + 2, ahead, words_ahead);
    // Multiplying stage s (reads one buffer) and converting stage s+1 (writes the other) are independent.  The two
    // wavefronts of a SIMD (w and w + 4) take them in opposite orders, so one's MFMAs run beside the other's vector
    // instructions instead of both queueing for the same pipe after every barrier.
    if (wave >= 4 && s + 1 < nstages)
      emit(s + 1, next, words_next);
    if (!idle) {
#pragma unroll
      for (int u = 0; u < kUnfoldSteps; ++u)
        multiply((s & 1) * kBufBytes + u * kStageBytes);
    }
    if (wave < 4 && s + 1 < nstages)
      emit(s + 1, next, words_next);
    // this wavefront's digits, words and row sums have reached LDS; no memory fence: it would wait for the loads of
    // stage s+2
    __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
    NBLA_BARRIER();
  };
  float va[16], vb[16];
  uint4_t wa, wb;
  gather(0, va, wa);
  if (nstages > 1)
    gather(1, vb, wb);
  emit(0, va, wa);
  __syncthreads();
  for (int s = 0; s < nstages; s += 2) {
    stage_step(s, va, wa, vb, wb);
    if (s + 1 < nstages)
      stage_step(s + 1, vb, wb, va, wa);
  }
}

template <int BM, int BN, int kWavesM, int kWavesN, int kWavesK, bool kSwap, int kUsed, bool kUnfold = false>
__device__ __forceinline__ void gemm_bits_body(GemmBitsArgs a, unsigned char *smem) {
#if defined(__HIP_DEVICE_COMPILE__) // the host pass only needs the launch stub; the body uses LDS address-space pointers
  static_assert(kUsed == 1 || kUsed == kDigits, "digits multiplied");
  static_assert(!kUnfold || (kSwap && kUsed == kDigits), "the unfolding product stores one lane per row, three digits");
  constexpr int kFirst = 0; // first digit (and accumulator) in use: digits kFirst .. kFirst + kUsed - 1
  constexpr int kWavesMN = kWavesM * kWavesN;
  constexpr int kWaves = kWavesMN * kWavesK;
  constexpr int MF = BM / kWavesM / 32;  // X fragments per wavefront (rows)
  constexpr int NF = BN / kWavesN / 32;  // B fragments per wavefront (columns)
  static_assert(BN % kWideGroup == 0 && (kWideGroup / 32) % NF == 0, "a wavefront's fragments share one wide group");
  constexpr int kASegs = BM / 32;            // row blocks per tile
  constexpr int kSegFrags = 2 * kUsed;       // fragments copied per row block per k step (2 k tiles x digits in use)
  constexpr int kSrcSegFrags = 2 * kDigits;  // fragments per row block per k step in the operand
  constexpr int kAFrags = kASegs * kSegFrags;
  constexpr int kBChunks = 2 * BN / kWideGroup; // 1 KiB chunks of packed words per k step (2 k tiles x wide groups)
  // One copy instruction moves 1 KiB (a fragment, or the words of one wide group); the kChunks copies of a k step
  // are dealt round-robin, so wavefronts below kExtra issue one more than the others.
  constexpr int kStepChunks = kAFrags + kBChunks;
  constexpr int kChunks = kStepChunks * kWavesK; // a stage holds kWavesK consecutive k steps
  constexpr int kPerWave = kChunks / kWaves, kExtra = kChunks % kWaves;
  constexpr int kABytes = kAFrags * kFragBytes;
  constexpr int kStepBytes = kStepChunks * kFragBytes;
  constexpr int kStageBytes = kStepBytes * kWavesK;
  // The LDS is sized for the three-digit stages.  One-digit stages are smaller, so more of them fit: the copies then
  // run further ahead, which is what a block that multiplies a third as much per k step needs to stay fed (at most
  // twelve stages, and few enough copies in flight for the 6-bit vmcnt).
  constexpr int kStagesFull = gemm_bits_stages(BM, BN, kWavesMN, kWavesK);
  constexpr int kLdsForStages = kStagesFull * gemm_bits_stage_bytes(BM, BN, kWavesK);
  constexpr int kStagesFit = kLdsForStages / kStageBytes < 12 ? kLdsForStages / kStageBytes : 12;
  constexpr int kStagesCnt = 63 / (kPerWave + 1) + 2; // (kStages - 2) * (kPerWave + 1) < 64
  constexpr int kStages = kUsed == kDigits ? kStagesFull : (kStagesFit < kStagesCnt ? kStagesFit : kStagesCnt);
  constexpr int kDepth = kStages - 1; // k steps in flight ahead of the one being multiplied
  // How many of the most recently issued k steps each wait may leave in flight: taken from the model of this loop's
  // order of copies, waits, barriers and LDS reads (copy_pipeline.hpp), which is also asserted safe as a whole.
  constexpr int kPrologueWait = pipeline::two_tile_prologue_wait(kStages, kDepth);
  constexpr int kLoopWait = pipeline::two_tile_loop_wait(kStages, kDepth);
  constexpr int kAheadWait = pipeline::read_ahead_loop_wait(kStages, kDepth); // the loop of one-digit rows
  static_assert(kPrologueWait >= 0 && kLoopWait >= 0 &&
                    pipeline::two_tile_safe(kStages, kDepth, kPrologueWait, kLoopWait),
                "the copy pipeline hands a buffer over too early");
  static_assert(pipeline::counter_fits(kPrologueWait, kPerWave + (kExtra ? 1 : 0)), "vmcnt is a 6-bit counter");

  if (a.split_steps > 0) {
    const int64_t begin = a.step_begin + (int64_t)blockIdx.y * a.split_steps;
    a.step_end = begin + a.split_steps < a.step_end ? begin + a.split_steps : a.step_end;
    a.step_begin = begin;
    a.y += (int64_t)blockIdx.y * a.M * a.N;
    a.use_sums = blockIdx.y == 0;
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave / kWavesMN, wmn = wave - wk * kWavesMN;
  const int wm = wmn % kWavesM, wn = wmn / kWavesM;

  // Tiles are walked in bands of kBand block rows, column by column inside a band: the blocks resident on an XCD at
  // one time then cover about kBand x kBand tiles, so its L2 serves each digit panel and each packed panel to
  // several blocks instead of streaming the whole packed operand once per block row.
  int64_t bm, bn;
  band_tile<8>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn);

  i32x16_t acc[kDigits][MF][NF];
#pragma unroll
  for (int d = 0; d < kDigits; ++d)
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int j = 0; j < NF; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[d][i][j][r] = 0;

  // Fragment fetch and the MFMA block of one k tile (t = 0, 1) of a staged step.
  auto read_a = [&](int buf_bytes, int t, uint4_t (&af)[MF][kUsed]) __attribute__((always_inline)) {
    const uint4_t *sa = reinterpret_cast<const uint4_t *>(smem + buf_bytes + wk * kStepBytes);
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int d = 0; d < kUsed; ++d)
        af[i][d] = sa[((wm * MF + i) * kSegFrags + t * kUsed + d) * 64 + lane];
  };
  const int frag0 = (wn * NF) % (kWideGroup / 32); // index of this wavefront's first column fragment in its group
  auto read_words = [&](int buf_bytes, int t, uint4_t &words) __attribute__((always_inline)) {
    const uint4_t *sb = reinterpret_cast<const uint4_t *>(smem + buf_bytes + wk * kStepBytes + kABytes);
    words = sb[(t * (BN / kWideGroup) + (wn * NF) / (kWideGroup / 32)) * 64 + lane];
  };
  // Bits -> bytes in {0, 2^F}: register i of column fragment F is word_i & (0x01010101 << F).
  uint32_t frag_mask[NF];
#pragma unroll
  for (int j = 0; j < NF; ++j) {
    frag_mask[j] = 0x01010101u << (frag0 + j);
    asm volatile("" : "+s"(frag_mask[j]));
  }
  auto mma = [&](const uint4_t (&af)[MF][kUsed], const uint4_t &words, auto j_begin, auto j_end) __attribute__((always_inline)) {
#pragma unroll
    for (int j = decltype(j_begin)::value; j < decltype(j_end)::value; ++j) {
      uint4_t bf;
      bf.x = words.x & frag_mask[j];
      bf.y = words.y & frag_mask[j];
      bf.z = words.z & frag_mask[j];
      bf.w = words.w & frag_mask[j];
#pragma unroll
      for (int d = 0; d < kUsed; ++d)
#pragma unroll
        for (int i = 0; i < MF; ++i) {
          const i32x4_t va = __builtin_bit_cast(i32x4_t, af[i][d]), vb = __builtin_bit_cast(i32x4_t, bf);
          acc[kFirst + d][i][j] =
              __builtin_amdgcn_mfma_i32_32x32x32_i8(kSwap ? vb : va, kSwap ? va : vb, acc[kFirst + d][i][j], 0, 0, 0);
        }
    }
  };
  typedef std::integral_constant<int, 0> J0;
  typedef std::integral_constant<int, 1> J1;
  typedef std::integral_constant<int, NF> JN;
  uint4_t af0[MF][kUsed], af1[MF][kUsed];
  uint4_t w0, w1;
  // A wavefront whose columns all lie past the end of the operand (last tile of a row of tiles) only takes part in
  // the copies and barriers: the matrix pipe of its SIMD is left to the other wavefront.
  const bool idle = a.n_begin + bn * BN + wn * NF * 32 >= a.n_end;
  // the epilogue's metadata (plain product): loaded here, written to LDS once the first copies have been issued
  constexpr int kThreadsAll = kWaves * 64;
  constexpr int kEpiOff = gemm_bits_lds_bytes(BM, BN, kWavesM, kWavesN, kWavesK);
  constexpr int kEpiCols = (BN + kThreadsAll - 1) / kThreadsAll;
  long long *epi_sums = reinterpret_cast<long long *>(smem + kEpiOff);
  int32_t *epi_shift = reinterpret_cast<int32_t *>(smem + kEpiOff + BM * 8);
  float *epi_alpha = reinterpret_cast<float *>(smem + kEpiOff + BM * 12), *epi_bias = epi_alpha + BN;
  long long meta_sum = 0;
  int32_t meta_shift = 0;
  float meta_alpha[kEpiCols], meta_bias[kEpiCols];
  if constexpr (!kUnfold) {
    if (tid < BM) {
      const int64_t m = bm * BM + tid;
      const int64_t ml = (m < a.row_blocks * kFragRows) ? m : 0; // row blocks past the operand are not stored
      meta_sum = a.use_sums ? a.sums[ml] : 0;
      meta_shift = a.shift[ml];
    }
#pragma unroll
    for (int c = 0; c < kEpiCols; ++c) {
      const int64_t n = a.n_begin + bn * BN + c * kThreadsAll + tid;
      const int64_t nc = n < a.N ? n : a.N - 1;
      meta_alpha[c] = (a.finish && a.alpha) ? a.alpha[nc] : 1.0f;
      meta_bias[c] = (a.finish && a.bias) ? a.bias[nc] : -0.0f;
    }
  }
  auto store_epilogue_metadata = [&]() __attribute__((always_inline)) {
    if (tid < BM) {
      epi_sums[tid] = meta_sum;
      epi_shift[tid] = meta_shift;
    }
#pragma unroll
    for (int c = 0; c < kEpiCols; ++c)
      if (c * kThreadsAll + tid < BN) {
        epi_alpha[c * kThreadsAll + tid] = meta_alpha[c];
        epi_bias[c * kThreadsAll + tid] = meta_bias[c];
      }
  };
  if constexpr (kUnfold) {
    unfold_main_loop<BM, BN, kWavesM, kWavesN, kWavesK, kStageBytes, kStepBytes, kABytes>(
        a, smem, bm, bn, wave, lane, idle, [&](int buf_bytes) __attribute__((always_inline)) {
          read_a(buf_bytes, 0, af0);
          read_words(buf_bytes, 0, w0);
          read_a(buf_bytes, 1, af1);
          read_words(buf_bytes, 1, w1);
          mma(af0, w0, J0(), JN());
          mma(af1, w1, J0(), JN());
        });
  } else {
    // Sources of this wavefront's copies.  Slot p of wavefront w copies chunk p * kWaves + w of every stage; the chunk is
    // described by a buffer resource that starts at the chunk's bytes in the first stage of this launch and ends with
    // its bytes in the last one, and by a scalar byte offset that advances by one stage per copy (the lane adds its own
    // 16 bytes).  The hardware range check (it covers the scalar offset too) turns a copy past the end (the copies run kDepth stages ahead of the last multiplication) into
    // zeros in LDS: no address is clamped in the loop.  Row blocks / wide groups past the end of the operand are
    // clamped here: their products land in rows / columns that are not stored.
    constexpr int kSlots = kPerWave + (kExtra ? 1 : 0);
    const int nstages = (int)((a.step_end - a.step_begin) / kWavesK);
    __amdgpu_buffer_rsrc_t rsrc[kSlots];
    uint32_t stage_bytes[kSlots]; // advance per stage
    uint32_t soff[kSlots];        // offset of the next stage inside the resource
    const uint32_t lane_bytes = lane * 16;
  #pragma unroll
    for (int p = 0; p < kSlots; ++p) {
      const int cs = p * kWaves + wave;                 // chunk of the stage
      const int kk = (cs / kStepChunks) % kWavesK;      // k step inside the stage
      const int c = cs - (cs / kStepChunks) * kStepChunks;
      const uint4_t *src;
      int64_t src_step; // advance per k step, in uint4
      if (c < kAFrags) {
        const int seg = c / kSegFrags, rem = c - seg * kSegFrags; // rem = (k tile of the step, digit in use)
        const int t = rem / kUsed, d = kFirst + rem - t * kUsed;
        int64_t rb = bm * kASegs + seg;
        if (rb >= a.row_blocks)
          rb = a.row_blocks - 1;
        src_step = kSrcSegFrags * 64;
        src = a.xd + (rb * a.x_k_tiles * kDigits + t * kDigits + d) * 64 + kk * src_step;
      } else {
        // packed words: chunk = (k tile of the step, wide group of the tile)
        const int cb = c - kAFrags;
        const int t = cb / (BN / kWideGroup);
        int64_t wg = a.n_begin / kWideGroup + bn * (BN / kWideGroup) + (cb - t * (BN / kWideGroup));
        if (wg >= a.wide_groups)
          wg = a.wide_groups - 1;
        src_step = 2 * a.wide_groups * 64;
        src = reinterpret_cast<const uint4_t *>(a.bits) + (t * a.wide_groups + wg) * 64 + kk * src_step;
      }
      stage_bytes[p] = (uint32_t)(src_step * kWavesK * 16); // the host checks that a launch's stages span < 4 GiB
      const uint32_t span = (uint32_t)(nstages - 1) * stage_bytes[p] + kFragBytes;
      // (every input is uniform; reading the address through the first lane tells the compiler so, which keeps the
      // resource in scalar registers)
      const uint64_t first = reinterpret_cast<uint64_t>(src + a.step_begin * src_step);
      const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(first >> 32)) << 32) |
                            (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
      rsrc[p] = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(base), 0,
                                                  __builtin_amdgcn_readfirstlane((int)span), 0x00020000);
      stage_bytes[p] = __builtin_amdgcn_readfirstlane((int)stage_bytes[p]);
      soff[p] = 0;
    }
    typedef __attribute__((address_space(3))) void lds_void_t;
    const int wave_lds = wave * kFragBytes;
    // issues this wavefront's kCount copies of the next stage into the LDS buffer at byte offset `buf_bytes`
    auto copy_next = [&](int buf_bytes, auto count_c) __attribute__((always_inline)) {
      constexpr int kCount = decltype(count_c)::value;
  #pragma unroll
      for (int p = 0; p < kCount; ++p) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc[p], (lds_void_t *)(smem + (wave_lds + buf_bytes) + p * kWaves * kFragBytes), 16, lane_bytes, soff[p], 0,
            0);
        soff[p] += stage_bytes[p];
      }
    };
    // waits until at most `steps` stages of this wavefront's copies (kCount each) are in flight
    auto wait_copies = [&](auto steps, auto count_c) __attribute__((always_inline)) {
      NBLA_WAIT_VMCNT(decltype(steps)::value * decltype(count_c)::value);
    };

    // Software pipeline.  One barrier per k step, in the middle of it.  A wavefront issues in order and an MFMA keeps
    // the matrix pipe busy for 32 cycles, so each half step is laid out by hand: the MFMAs of the first column
    // fragment go first, the LDS reads of the next k tile (and the copies of a later k step) are issued in their
    // shadow, and the remaining MFMAs cover the latency.  sched_barrier pins that order.
    // Everything that is not an MFMA is kept short, because a wavefront cannot feed the matrix pipe while it works
    // through scalar and address instructions: the copies are bounds-checked buffer loads whose addresses advance by
    // one scalar add each; the number of copies a wavefront issues per stage (kPerWave, or one more for the first
    // kExtra wavefronts) is a compile-time constant of its copy of the loop; the ring position is kept as three byte
    // offsets that rotate; the loop counter is 32 bits wide.
    auto run = [&](auto count_c) __attribute__((always_inline)) {
  #pragma unroll
      for (int d = 0; d < kDepth; ++d)
        copy_next(d * kStageBytes, count_c);
      store_epilogue_metadata(); // its loads were issued before the copies: waiting for them leaves the copies in flight
      wait_copies(std::integral_constant<int, kPrologueWait>(), count_c);
      NBLA_BARRIER();
      read_words(0, 0, w0);
      read_a(0, 0, af0);
      // byte offsets of the LDS buffers of step ks (`cur`), of step ks-1 = that of step ks+kDepth (`prev`)
      int cur = 0, prev = (kStages - 1) * kStageBytes;
      if (kUsed == 1 && !idle) {
        // One-digit rows: a step has a third of the MFMAs, too few to cover an LDS read issued in the same step, and
        // a third of the operand registers.  So both k tiles of step ks+1 are read at the top of step ks (after the
        // barrier that says they have landed everywhere) and multiplied one step later, from registers.
        static_assert(pipeline::read_ahead_safe(kStages, kDepth, kPrologueWait, kAheadWait),
                      "the copy pipeline hands a buffer over too early");
        read_words(0, 1, w1);
        read_a(0, 1, af1);
        for (int left = nstages; left > 0; --left) {
          const int next = (cur + kStageBytes == kStages * kStageBytes) ? 0 : cur + kStageBytes;
          uint4_t an0[MF][kUsed], an1[MF][kUsed], wn0, wn1;
          wait_copies(std::integral_constant<int, kAheadWait>(), count_c);
          // this wavefront's reads of step ks (issued a step ago) have returned: after the barrier another wavefront
          // may send a copy into a buffer that holds an older step only, but the wait costs nothing here
          __builtin_amdgcn_s_waitcnt(0xc07f);
          NBLA_BARRIER();
          if (left > 1) {
            read_words(next, 0, wn0);
            read_a(next, 0, an0);
            read_words(next, 1, wn1);
            read_a(next, 1, an1);
          }
          __builtin_amdgcn_sched_barrier(0);
          mma(af0, w0, J0(), JN());
          mma(af1, w1, J0(), JN());
          __builtin_amdgcn_sched_barrier(0);
          copy_next(prev, count_c);
          if (left > 1) {
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
              for (int d = 0; d < kUsed; ++d)
                af0[i][d] = an0[i][d], af1[i][d] = an1[i][d];
            w0 = wn0, w1 = wn1;
          }
          prev = cur;
          cur = next;
        }
        return;
      }
      if (idle) {
        for (int left = nstages; left > 0; --left) {
          wait_copies(std::integral_constant<int, kLoopWait>(), count_c);
          NBLA_BARRIER();
          copy_next(prev, count_c);
          prev = cur;
          cur = (cur + kStageBytes == kStages * kStageBytes) ? 0 : cur + kStageBytes;
        }
        return;
      }
      // Three-digit rows.  Between two MFMAs a wavefront can issue a few other instructions without starving the
      // matrix pipe, but not a batch of them: the LDS reads of the next k tile and the copies of a later step are
      // therefore dealt out one per MFMA (sched_group_barrier: 0x008 = MFMA, 0x100 = LDS read, 0x020 = the copies'
      // buffer loads) instead of standing together between two groups of MFMAs.  A wavefront that has its SIMD to
      // itself (its neighbour is in its prologue or epilogue) gains most: 0.421 -> 0.400 ms for the launch with one
      // block per CU, 0.360 -> 0.354 ms with two.
      constexpr int kCopies = decltype(count_c)::value;
      constexpr int kReads = MF * kUsed + 1, kMfmas = MF * NF * kUsed;
      static_assert(kUsed == 1 || kReads + kCopies <= kMfmas, "more reads and copies than MFMAs to deal them out to");
      for (int left = nstages; left > 0; --left) {
        const int next = (cur + kStageBytes == kStages * kStageBytes) ? 0 : cur + kStageBytes;
        // tile 0 runs; tile 1 (same stage: it landed with tile 0) is fetched
        read_a(cur, 1, af1);
        read_words(cur, 1, w1);
        mma(af0, w0, J0(), JN());
#pragma unroll
        for (int i = 0; i < kReads; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmas - kReads, 0);
        __builtin_amdgcn_sched_barrier(0);
        // step ks+1 has landed: the copies issued so far reach step ks+kDepth-1, so at most the kDepth-2 (= kLoopWait)
        // steps behind ks+1 may still be in flight; every wavefront is done with the buffer of step ks-1
        wait_copies(std::integral_constant<int, kLoopWait>(), count_c);
        NBLA_BARRIER();
        // tile 1 runs; the copy of step ks+kDepth is issued; tile 0 of step ks+1 is fetched
        copy_next(prev, count_c);
        read_words(next, 0, w0);
        read_a(next, 0, af0);
        mma(af1, w1, J0(), JN());
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 1);
        }
#pragma unroll
        for (int i = 0; i < kReads; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmas - kReads - kCopies, 1);
        __builtin_amdgcn_sched_barrier(0);
        prev = cur;
        cur = next;
      }
    };
    if (kExtra && wave < kExtra)
      run(std::integral_constant<int, kPerWave + 1>());
    else
      run(std::integral_constant<int, kPerWave>());
  }
  NBLA_WAIT_VMCNT(0);

  if (kWavesK > 1) {
    // Exact sum of the k groups' accumulators through LDS (the staging buffers are free now), one digit at a time:
    // groups 1.. store, group 0 adds.
    uint4_t *red = reinterpret_cast<uint4_t *>(smem);
    constexpr int kRegs4 = MF * NF * 4; // uint4 per lane per digit
#pragma unroll
    for (int d = kFirst; d < kFirst + kUsed; ++d) {
      NBLA_BARRIER();
      if (wk > 0 && !idle) {
        uint4_t *dst = red + (size_t)((wk - 1) * kWavesMN + wmn) * kRegs4 * 64 + lane;
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
          for (int j = 0; j < NF; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              uint4_t v;
              v.x = acc[d][i][j][4 * q + 0], v.y = acc[d][i][j][4 * q + 1];
              v.z = acc[d][i][j][4 * q + 2], v.w = acc[d][i][j][4 * q + 3];
              dst[((i * NF + j) * 4 + q) * 64] = v;
            }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): the stores have reached LDS
      NBLA_BARRIER();
      if (wk == 0 && !idle) {
#pragma unroll
        for (int g = 1; g < kWavesK; ++g) {
          const uint4_t *srcp = red + (size_t)((g - 1) * kWavesMN + wmn) * kRegs4 * 64 + lane;
#pragma unroll
          for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int j = 0; j < NF; ++j)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const uint4_t v = srcp[((i * NF + j) * 4 + q) * 64];
                acc[d][i][j][4 * q + 0] += (int)v.x, acc[d][i][j][4 * q + 1] += (int)v.y;
                acc[d][i][j][4 * q + 2] += (int)v.z, acc[d][i][j][4 * q + 3] += (int)v.w;
              }
        }
      }
    }
    if (wk > 0)
      return;
  }

  // Epilogue.  Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
  // column l%32 of the 32x32 fragment; rows are m and columns n, or the reverse
  // under kSwap.
  // Everything an output element needs besides its accumulators (row sums and shift, alpha, bias) is loaded into
  // registers before the stores of the group it belongs to: the compiler cannot move a load across a store to y.
  const int col_in_frag = lane & 31, row_half = lane >> 5;
  // start of output row m (32-bit division: M and inner are below 2^31)
  auto row_ptr = [&](int64_t m) {
    const uint32_t mu = (uint32_t)m, in = (uint32_t)a.inner;
    const int64_t off = (in == 1u) ? m * a.outer_stride : (int64_t)(mu / in) * a.outer_stride + (mu % in);
    return a.y + off;
  };
  // The stores run in two copies, with and without reading y back first (k chunks after the first add to it): with
  // the loads of the accumulating form anywhere in the same code the compiler waits for all outstanding memory
  // operations before every output (the loads might be pending), and stores are outstanding memory operations, so
  // each store would wait for the one before it.  Likewise with and without the bound checks a block on the edge
  // of the output needs (a branch on the execution mask per store).
  auto store_tile = [&](auto accumulate_c, auto inside_c) __attribute__((always_inline)) {
    constexpr bool kAcc = decltype(accumulate_c)::value;
    constexpr bool kInside = decltype(inside_c)::value; // every row and column of the block is stored: no checks
    // al is 1 and bi is -0 where there is no alpha / bias (or this is not the last k chunk): exact identities
    auto finish = [&](float v, float prev, float al, float bi) {
      if (kAcc)
        v = prev + v;
      v = v * al;
      v = v + bi;
      return v;
    };
    FragScale fs[NF];
  #pragma unroll
    for (int j = 0; j < NF; ++j)
      fs[j] = frag_scale(frag0 + j);
    if (!kSwap) {
      const int64_t ncol0 = a.n_begin + bn * BN + wn * NF * 32 + col_in_frag;
      float al[NF], bi[NF];
  #pragma unroll
      for (int j = 0; j < NF; ++j) {
        al[j] = epi_alpha[wn * NF * 32 + col_in_frag + 32 * j];
        bi[j] = epi_bias[wn * NF * 32 + col_in_frag + 32 * j];
      }
  #pragma unroll
      for (int i = 0; i < MF; ++i) {
        const int64_t m0 = bm * BM + (wm * MF + i) * 32 + 4 * row_half;
  #pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          // rows m0 + 8 rq + 0..3 (the metadata arrays are padded to whole row blocks)
          const int64_t mq = m0 + 8 * rq;
          const int rl = (wm * MF + i) * 32 + 4 * row_half + 8 * rq; // the same rows inside the block
          const i32x4_t sum01 = *reinterpret_cast<const i32x4_t *>(epi_sums + rl); // two int64 as (lo, hi) words
          const i32x4_t sum23 = *reinterpret_cast<const i32x4_t *>(epi_sums + rl + 2);
          i32x4_t sh = *reinterpret_cast<const i32x4_t *>(epi_shift + rl);
  #pragma unroll
          for (int e = 0; e < 4; ++e)
            sh[e] = plain_shift(sh[e]); // one-digit rows store their shift with a bias (kBadRow is negative: unchanged)
          // sum = s_hi * 65536 + s_lo with s_lo in [0, 65536)
          const uint32_t lo_w[4] = {(uint32_t)sum01.x, (uint32_t)sum01.z, (uint32_t)sum23.x, (uint32_t)sum23.z};
          const int hi_w[4] = {sum01.y, sum01.w, sum23.y, sum23.w};
          int s_hi[4], s_lo[4], neg_sh[4];
          float hi_scale[4];
  #pragma unroll
          for (int e = 0; e < 4; ++e) {
            s_hi[e] = (int)((lo_w[e] >> 16) | ((uint32_t)hi_w[e] << 16));
            s_lo[e] = (int)(lo_w[e] & 0xffffu);
            neg_sh[e] = row_neg_shift(sh[e]);
            hi_scale[e] = row_hi_scale(sh[e]);
          }
  #pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * rq + e;
            if (!kInside && mq + e >= a.M)
              continue;
            if (sh[e] == kBadRow && a.keep_bad_rows) // the caller has computed this row
              continue;
            float *row = row_ptr(mq + e) + ncol0 * a.n_stride;
            float prev[NF];
            if (kAcc) {
  #pragma unroll
              for (int j = 0; j < NF; ++j)
                prev[j] = (kInside || ncol0 + 32 * j < a.n_end) ? row[32 * j * a.n_stride] : 0.0f;
            }
  #pragma unroll
            for (int j = 0; j < NF; ++j) {
              float v = finish_dot(acc[0][i][j][r], acc[1][i][j][r], acc[2][i][j][r], s_hi[e], s_lo[e], neg_sh[e],
                                   hi_scale[e], fs[j]);
              v = finish(v, prev[j], al[j], bi[j]);
              if (kInside || ncol0 + 32 * j < a.n_end)
                __builtin_nontemporal_store(v, row + 32 * j * a.n_stride);
            }
          }
        }
      }
    } else {
  #pragma unroll
      for (int i = 0; i < MF; ++i) {
        const int64_t m = bm * BM + (wm * MF + i) * 32 + col_in_frag;
        if (!kInside && m >= a.M)
          continue;
        long long sum;
        int sh;
        if constexpr (kUnfold) { // the block's own rows, left in LDS by unfold_main_loop
          constexpr int kMetaOff = unfold_meta_off(BM, BN, kWavesM, kWavesN, kWavesK);
          sum = reinterpret_cast<const long long *>(smem + kMetaOff)[m - bm * BM];
          sh = reinterpret_cast<const int32_t *>(smem + kMetaOff + 384)[m - bm * BM];
        } else {
          sum = epi_sums[m - bm * BM];
          sh = plain_shift(epi_shift[m - bm * BM]);
        }
        const int s_hi = (int)(sum >> 16), s_lo = (int)(sum & 0xffff);
        if (sh == kBadRow && a.keep_bad_rows) // the caller has computed this row
          continue;
        const int neg_sh = row_neg_shift(sh);
        const float hi_scale = row_hi_scale(sh);
        float *row = row_ptr(m);
  #pragma unroll
        for (int j = 0; j < NF; ++j) {
  #pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            const int64_t n0 = a.n_begin + bn * BN + (wn * NF + j) * 32 + 4 * row_half + 8 * rq;
            float al[4], bi[4], prev[4];
  #pragma unroll
            for (int e = 0; e < 4; ++e) {
              if constexpr (kUnfold) { // left in LDS by unfold_main_loop (1 and -0 where there is no alpha / bias)
                constexpr int kMetaOff = unfold_meta_off(BM, BN, kWavesM, kWavesN, kWavesK);
                const float *s_alpha = reinterpret_cast<const float *>(smem + kMetaOff + 512 + 64 * 16);
                const int col = (int)(n0 + e - a.n_begin - bn * BN);
                al[e] = s_alpha[col];
                bi[e] = s_alpha[256 + col];
              } else {
                const int col = (wn * NF + j) * 32 + 4 * row_half + 8 * rq + e;
                al[e] = epi_alpha[col];
                bi[e] = epi_bias[col];
              }
            }
            float *p = row + n0 * a.n_stride;
            if (kAcc) {
  #pragma unroll
              for (int e = 0; e < 4; ++e)
                prev[e] = (kInside || n0 + e < a.n_end) ? p[e * a.n_stride] : 0.0f;
            }
  #pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = 4 * rq + e;
              float v = finish_dot(acc[0][i][j][r], acc[1][i][j][r], acc[2][i][j][r], s_hi, s_lo, neg_sh, hi_scale,
                                   fs[j]);
              v = finish(v, prev[e], al[e], bi[e]);
              if (kInside || n0 + e < a.n_end)
                __builtin_nontemporal_store(v, p + e * a.n_stride);
            }
          }
        }
      }
    }
  };
  const bool inside = (bm + 1) * BM <= a.M && a.n_begin + (bn + 1) * BN <= a.n_end;
  if (a.accumulate) {
    if (inside)
      store_tile(std::true_type(), std::true_type());
    else
      store_tile(std::true_type(), std::false_type());
  } else {
    if (inside)
      store_tile(std::false_type(), std::true_type());
    else
      store_tile(std::false_type(), std::false_type());
  }
#endif
}

template <int BM, int BN, int kWavesM, int kWavesN, int kWavesK, bool kSwap>
__global__ __launch_bounds__(kWavesM *kWavesN *kWavesK * 64, (kWavesM * kWavesN * kWavesK >= 8 ? 1 : 2)) void gemm_bits_kernel(GemmBitsArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  if (a.skip_if && *a.skip_if != 0) // uniform over the grid
    return;
  // Are all rows of this block's row blocks one-digit rows?  (Same tile mapping as the body; rows past the operand
  // are clamped to its last row, as the copies are.)
  int64_t bm, bn;
  band_tile<8>(blockIdx.x, a.blocks_m, a.blocks_n, bm, bn);
  const int64_t rows = a.row_blocks * kFragRows;
  bool one = true;
  for (int r = threadIdx.x; r < BM; r += kWavesM * kWavesN * kWavesK * 64) {
    const int64_t m = bm * BM + r;
    one = one && one_digit_row(a.shift[m < rows ? m : rows - 1]);
  }
  if (__syncthreads_and(one))
    gemm_bits_body<BM, BN, kWavesM, kWavesN, kWavesK, kSwap, 1>(a, smem);
  else
    gemm_bits_body<BM, BN, kWavesM, kWavesN, kWavesK, kSwap, kDigits>(a, smem);
}

// The convolution's product with the unfold fused in (unfold_main_loop): one block per 32 windows and 256 output
// channels, eight wavefronts (four column pairs x two k groups).
__global__ __launch_bounds__(512, 1) void gemm_bits_unfold_kernel(GemmBitsArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  gemm_bits_body<32, 256, 1, 4, 2, true, kDigits, true>(a, smem);
}

// Measurement aid: while armed, the calling thread's launches of the product carry a pair of events that the runtime
// stamps with the dispatch's own begin and end (hipExtLaunchKernelGGL), i.e. the kernel's duration as a profiler
// sees it, without the queue bubbles that event records between launches add.
struct KernelTimer {
  std::vector<hipEvent_t> start, stop;
  size_t used = 0;
};
thread_local KernelTimer t_timer;

void kernel_timer_release() {
  for (hipEvent_t e : t_timer.start)
    (void)hipEventDestroy(e);
  for (hipEvent_t e : t_timer.stop)
    (void)hipEventDestroy(e);
  t_timer.start.clear(), t_timer.stop.clear(), t_timer.used = 0;
}

template <int BM, int BN, int kWavesM, int kWavesN, int kWavesK, bool kSwap>
int launch_tile(const GemmBitsArgs &args, hipStream_t stream, unsigned splits = 1) {
  constexpr int kThreads = kWavesM * kWavesN * kWavesK * 64;
  constexpr int kSmem = gemm_bits_lds_bytes(BM, BN, kWavesM, kWavesN, kWavesK) + gemm_bits_epilogue_bytes(BM, BN);
  // the kernel is named at each launch, not held in a pointer: a launch through a pointer is an indirect call of
  // the host-side stub, which -fsanitize=function builds instrument (and then drop)
#define NBLA_GEMM_BITS_KERNEL gemm_bits_kernel<BM, BN, kWavesM, kWavesN, kWavesK, kSwap>
  static std::atomic<uint64_t> configured{0};
  const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(&NBLA_GEMM_BITS_KERNEL), kSmem, configured,
                                   "hipFuncSetAttribute(gemm_bits LDS size)");
  if (rc)
    return rc;
  GemmBitsArgs a = args;
  a.blocks_m = ceil_div(a.M, BM);
  a.blocks_n = ceil_div(a.n_end - a.n_begin, BN);
  const dim3 grid((unsigned)(a.blocks_m * a.blocks_n), splits);
  if (t_timer.used < t_timer.start.size()) {
    hipExtLaunchKernelGGL((NBLA_GEMM_BITS_KERNEL), grid, dim3(kThreads), kSmem, stream, t_timer.start[t_timer.used],
                          t_timer.stop[t_timer.used], 0, a);
    ++t_timer.used;
  } else {
    hipLaunchKernelGGL((NBLA_GEMM_BITS_KERNEL), grid, dim3(kThreads), kSmem, stream, a);
  }
#undef NBLA_GEMM_BITS_KERNEL
  NBLA_HIP_LAUNCH_CHECK("gemm_bits");
  return NBLA_HIP_OK;
}

// Tile choice.  A wavefront owns 32x128 outputs (its three accumulator sets take 192 registers), so eight
// wavefronts fill a CU.  Blocks of four wavefronts (one per SIMD), two blocks per CU, measured best: the barrier
// couples only four wavefronts and one block's prologue / epilogue overlaps the other's main loop.  The packed
// operand costs 1/24 of the digit operand's bytes per element, so the block tile is one row block high and wide
// (32x512) to keep the global -> LDS traffic lowest; narrow outputs take 32x256 blocks of two wavefronts, and
// outputs of at most 256 such tiles use eight wavefronts per 32x256 tile, four k groups of two; outputs of at most
// 256 wide tiles (every CU would hold a single block of four wavefronts) eight wavefronts per 32x512 tile, two k
// groups of four.
// Splits of the contraction over blocks for an output of `tiles` 32x256 tiles and `steps` k steps: as many as give
// every CU a block, at least eight k steps (two rounds of the four k groups) each; 1 = no split.
inline int64_t bit_product_splits(int64_t tiles, int64_t steps) {
  if (tiles * 2 > 256 || steps < 16)
    return 1;
  const int64_t by_cus = 256 / tiles, by_k = steps / 8;
  return by_cus < by_k ? by_cus : by_k;
}

// y (+)= (sum over the splits, in split order) (* alpha) (+ bias): the order of operations of the kernel's epilogue.
__global__ __launch_bounds__(256) void gemm_bits_split_sum(const float *__restrict__ partial, int splits, int64_t M,
                                                           int64_t N, float *__restrict__ y, int64_t inner,
                                                           int64_t outer_stride, int64_t n_stride,
                                                           const float *__restrict__ alpha,
                                                           const float *__restrict__ bias, int accumulate,
                                                           const int32_t *__restrict__ keep_shift,
                                                           const int *__restrict__ skip_if) {
  if (skip_if && *skip_if != 0)
    return;
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / N, n = i - m * N;
    if (keep_shift && keep_shift[m] == kBadRow) // the caller has computed this row
      continue;
    float v = partial[i];
    for (int z = 1; z < splits; ++z)
      v += partial[(int64_t)z * total + i];
    const int64_t q = m / inner;
    float *dst = y + q * outer_stride + (m - q * inner) + n * n_stride;
    if (accumulate)
      v = *dst + v;
    if (alpha)
      v = v * alpha[n];
    if (bias)
      v = v + bias[n];
    *dst = v;
  }
}

template <bool kSwap> int dispatch(const GemmBitsArgs &a, hipStream_t stream, void *split_ws, size_t split_ws_bytes) {
  const int64_t narrow_tiles = ceil_div(a.M, 32) * ceil_div(a.N, 256);
  if (!kSwap && split_ws) {
    int64_t splits = bit_product_splits(narrow_tiles, a.step_end - a.step_begin);
    while (splits > 1 && (size_t)splits * a.M * a.N * sizeof(float) > split_ws_bytes)
      --splits;
    if (splits > 1) {
      GemmBitsArgs part = a;
      part.split_steps = ceil_div(ceil_div(a.step_end - a.step_begin, splits), 4) * 4; // whole rounds of the k groups
      splits = ceil_div(a.step_end - a.step_begin, part.split_steps);
      part.y = static_cast<float *>(split_ws);
      part.inner = 1, part.outer_stride = a.N, part.n_stride = 1;
      part.accumulate = 0, part.finish = 0, part.keep_bad_rows = 0;
      int rc = launch_tile<32, 256, 1, 2, 4, kSwap>(part, stream, (unsigned)splits);
      if (rc)
        return rc;
      int64_t blocks = ceil_div(a.M * a.N, 256);
      if (blocks > 4096)
        blocks = 4096;
      hipLaunchKernelGGL(gemm_bits_split_sum, dim3((unsigned)blocks), dim3(256), 0, stream,
                         static_cast<const float *>(split_ws), (int)splits, a.M, a.N, a.y, a.inner, a.outer_stride,
                         a.n_stride, a.finish ? a.alpha : nullptr, a.finish ? a.bias : nullptr, a.accumulate,
                         a.keep_bad_rows ? a.shift : nullptr, a.skip_if);
      NBLA_HIP_LAUNCH_CHECK("gemm_bits_split_sum");
      return NBLA_HIP_OK;
    }
  }
  if (narrow_tiles <= 256) // too few tiles for the CUs: four k groups per tile
    return launch_tile<32, 256, 1, 2, 4, kSwap>(a, stream);
  if (a.N > 256 && ceil_div(a.M, 32) * ceil_div(a.N, 512) <= 256) // one wide tile per CU at most: two k groups
    return launch_tile<32, 512, 1, 4, 2, kSwap>(a, stream);
  if (a.N > 256)
    return launch_tile<32, 512, 1, 4, 1, kSwap>(a, stream);
  return launch_tile<32, 256, 1, 2, 1, kSwap>(a, stream);
}

} // namespace

int launch_gemm_bits(const void *xdigits, const uint32_t *bits, const float *alpha, const float *bias, float *y,
                     int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride, int64_t n_stride,
                     bool swap_out, hipStream_t stream, bool accumulate, void *split_ws, size_t split_ws_bytes,
                     bool keep_bad_rows, const int *skip_if) {
  if (M <= 0 || K <= 0 || N <= 0 || inner <= 0 || M > 0x7fffffffll || inner > 0x7fffffffll)
    return fail(NBLA_HIP_ERR_VALUE, "invalid GEMM shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  if (!aligned16(xdigits) || !aligned16(bits))
    return fail(NBLA_HIP_ERR_MEMORY, "GEMM operands must be 16-byte aligned.");
  // the copies address one launch's share of the packed operand (at most kChunkK / 32 k tiles) with 32-bit offsets
  if (bits_wide_groups(N) * kFragBytes * (kChunkK / kTileK) >= (int64_t)0xffffffffll)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "bit-weight product: more than %lld output columns are not supported.",
                (long long)(0xffffffffll / (kFragBytes * (kChunkK / kTileK)) * kWideGroup));
  int rc = ensure_init();
  if (rc)
    return rc;
  const DigitOperand d = digit_operand(M, K);
  const char *base = static_cast<const char *>(xdigits);
  GemmBitsArgs a;
  a.xd = reinterpret_cast<const uint4_t *>(base);
  a.shift = reinterpret_cast<const int32_t *>(base + d.shift_off);
  a.bits = bits;
  a.alpha = alpha;
  a.bias = bias;
  a.y = y;
  a.M = M;
  a.N = N;
  a.n_begin = 0;
  a.n_end = N;
  a.row_blocks = d.row_blocks;
  a.x_k_tiles = d.k_tiles;
  a.wide_groups = bits_wide_groups(N);
  a.blocks_m = a.blocks_n = 0;
  a.split_steps = 0;
  a.use_sums = 1;
  a.keep_bad_rows = keep_bad_rows ? 1 : 0;
  a.skip_if = skip_if;
  a.shift_out = nullptr;
  a.ux = nullptr;
  a.ugrp = 0;
  a.inner = inner;
  a.outer_stride = outer_stride;
  a.n_stride = n_stride;
  // one launch per chunk of kChunkK columns of x: the int32 accumulators of a chunk cannot overflow, and the fp32
  // partial results of the chunks are added up in y
  const int64_t steps_per_chunk = kChunkK / (2 * kTileK), steps = d.k_tiles / 2;
  for (int64_t c = 0; c < d.chunks; ++c) {
    a.sums = reinterpret_cast<const long long *>(base + d.sum_off) + c * d.rows;
    a.step_begin = c * steps_per_chunk;
    a.step_end = (a.step_begin + steps_per_chunk < steps) ? a.step_begin + steps_per_chunk : steps;
    a.accumulate = c > 0 || accumulate;
    a.finish = c + 1 == d.chunks;
    rc = swap_out ? dispatch<true>(a, stream, nullptr, 0) : dispatch<false>(a, stream, split_ws, split_ws_bytes);
    if (rc)
      return rc;
  }
  return NBLA_HIP_OK;
}

// LDS of the unfolding product: two stage buffers (or the k groups' exchange), the rows' metadata, the column table
static size_t unfold_lds_bytes(int64_t Kg) {
  return (size_t)unfold_meta_off(32, 256, 1, 4, 2) + kUnfoldMetaBytes + (size_t)bits_packed_k_tiles(Kg) * kTileK * 8;
}
static_assert(kUnfoldSteps * 2 * 2 == 8, "the packed operand's k tiles come in multiples of eight: whole stages");

bool gemm_bits_unfold_applies(const ConvGeom &g) {
  // x below 2 GiB (its elements are read through one buffer descriptor, at 32-bit byte offsets whose upper half
  // means "nowhere"), 32-bit positions inside one output map, 16-bit tap displacements (as the stand-alone unfold
  // kernel), one k chunk, and a column table that fits the LDS beside the stages
  bool fits = g.outer * g.C * g.in_sp_size * 4 < ((int64_t)1 << 31) && g.out_sp_size < ((int64_t)1 << 31) &&
              g.Kg <= kChunkK && g.M < ((int64_t)1 << 31) - 64;
  for (int i = 0; i < kMaxSpatial; ++i)
    fits = fits && (int64_t)(g.k[i] - 1) * g.dil[i] < 65536;
  return fits && g.k_size <= 64 && unfold_lds_bytes(g.Kg) <= 144 * 1024; // the taps of a row are a 64-bit mask
}

int launch_gemm_bits_unfold(const float *x, const ConvGeom &g, int64_t grp, const uint32_t *bits, const float *alpha,
                            const float *bias, float *y, hipStream_t stream, int32_t *row_shift) {
  if (!gemm_bits_unfold_applies(g))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "the fused unfold product does not cover this geometry.");
  if (!aligned16(bits))
    return fail(NBLA_HIP_ERR_MEMORY, "GEMM operands must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  const size_t lds = unfold_lds_bytes(g.Kg);
  static std::atomic<uint64_t> configured{0};
  rc = allow_dynamic_lds(reinterpret_cast<const void *>(gemm_bits_unfold_kernel), 144 * 1024, configured,
                         "hipFuncSetAttribute(gemm_bits_unfold LDS size)");
  if (rc)
    return rc;
  const int64_t hw = g.out_sp_size;
  GemmBitsArgs a;
  a.xd = nullptr;
  a.sums = nullptr;
  a.shift = nullptr;
  a.bits = bits;
  a.alpha = alpha;
  a.bias = bias;
  a.y = y;
  a.M = g.M;
  a.N = g.Og;
  a.n_begin = 0;
  a.n_end = g.Og;
  a.row_blocks = split_row_blocks(g.M);
  a.x_k_tiles = bits_packed_k_tiles(g.Kg);
  a.wide_groups = bits_wide_groups(g.Og);
  a.step_begin = 0;
  a.step_end = a.x_k_tiles / 2;
  a.blocks_m = a.row_blocks;
  a.blocks_n = a.wide_groups;
  a.inner = hw;
  a.outer_stride = g.O * hw;
  a.n_stride = hw;
  a.accumulate = 0;
  a.finish = 1;
  a.split_steps = 0;
  a.use_sums = 1;
  a.keep_bad_rows = 0;
  a.skip_if = nullptr;
  a.shift_out = row_shift;
  a.ux = x;
  a.ug = g;
  a.ugrp = grp;
  hipLaunchKernelGGL(gemm_bits_unfold_kernel, dim3((unsigned)(a.blocks_m * a.blocks_n)), dim3(512), lds, stream, a);
  NBLA_HIP_LAUNCH_CHECK("gemm_bits_unfold");
  return NBLA_HIP_OK;
}

size_t gemm_bits_split_bytes(int64_t M, int64_t K, int64_t N) {
  const int64_t steps = digit_k_tiles(K < kChunkK ? K : kChunkK) / 2;
  const int64_t s = bit_product_splits(ceil_div(M, 32) * ceil_div(N, 256), steps);
  return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" size_t nbla_hip_gemm_bits_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  return M > 0 && K > 0 && N > 0 ? round_up(gemm_bits_split_bytes(M, K, N), 256) : 0;
}

extern "C" int nbla_hip_gemm_bits_f32(const void *xdigits, const uint32_t *bits, const float *alpha, const float *bias,
                                      float *y, int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride,
                                      int64_t n_stride, void *workspace, size_t workspace_bytes, void *stream) {
  // m-contiguous outputs (n_stride != 1) store from the transposed accumulator tile
  return launch_gemm_bits(xdigits, bits, alpha, bias, y, M, K, N, inner, outer_stride, n_stride, n_stride != 1,
                          as_stream(stream), false, workspace, workspace_bytes);
}

extern "C" int nbla_hip_gemm_bits_timer_arm(int launches) {
  if (launches < 1 || launches > 65536)
    return fail(NBLA_HIP_ERR_VALUE, "product timer: between 1 and 65536 launches.");
  const int rc = ensure_init();
  if (rc)
    return rc;
  kernel_timer_release();
  for (int i = 0; i < launches; ++i) {
    hipEvent_t a = nullptr, b = nullptr;
    hipError_t e = hipEventCreate(&a);
    if (e == hipSuccess)
      e = hipEventCreate(&b);
    if (e != hipSuccess) {
      if (a)
        (void)hipEventDestroy(a);
      kernel_timer_release();
      return fail_hip(e, "hipEventCreate");
    }
    t_timer.start.push_back(a), t_timer.stop.push_back(b);
  }
  return NBLA_HIP_OK;
}

extern "C" int nbla_hip_gemm_bits_timer_read(int *launches, double *mean_ms, double *min_ms, double *max_ms) {
  const size_t n = t_timer.used;
  double sum = 0.0, lo = 0.0, hi = 0.0;
  for (size_t i = 0; i < n; ++i) {
    float ms = 0.0f;
    hipError_t e = hipEventSynchronize(t_timer.stop[i]);
    if (e == hipSuccess)
      e = hipEventElapsedTime(&ms, t_timer.start[i], t_timer.stop[i]);
    if (e != hipSuccess) {
      kernel_timer_release();
      return fail_hip(e, "product timer");
    }
    sum += ms;
    lo = (i == 0 || ms < lo) ? ms : lo, hi = (i == 0 || ms > hi) ? ms : hi;
  }
  kernel_timer_release();
  if (launches)
    *launches = (int)n;
  if (mean_ms)
    *mean_ms = n ? sum / (double)n : 0.0;
  if (min_ms)
    *min_ms = lo;
  if (max_ms)
    *max_ms = hi;
  return NBLA_HIP_OK;
}
