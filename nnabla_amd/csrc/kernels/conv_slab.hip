// Binary convolution forward on the int8 matrix cores with the unfold done by addressing (convolution.cpp:161-197 and
// unfold_to_patches.cpp:103-194 unfold x into a matrix [positions, channels x taps] and multiply it by the weights;
// here that matrix is never formed, not even in LDS).
//
// A block owns up to 32 consecutive output positions of one sample and 256 output channels.  Every input position
// ("pixel") that one of its windows touches lies in one run [lo, hi] of the flattened input map; the block reads that
// run of all the group's channels once (coalesced along the positions), turns every value into four balanced
// base-256 int8 digits under ONE power-of-two scale for the whole slab, and keeps the digits in LDS pixel by pixel:
//     slab[pixel 0..npix][channel tile of 32][digit 0..3][32 channels]   (pixel 0 is all zeros: the taps that fall
//                                                                         outside the input)
// The contraction runs over k' = (tap, channel) instead of the reference's (channel, tap): exact integer sums do not
// depend on the order, and in this order the sixteen k-slots of a lane of the i8 MFMA operand are sixteen
// consecutive channels of ONE pixel -- one 16-byte LDS read at (pixel of the lane's window under that tap) + channel
// offset.  So a value is converted once per block (not once per window that holds it: nine times for a 3 x 3 kernel),
// nothing is gathered element by element, and the main loop is LDS reads, one load of packed weight bits per k tile
// and MFMAs, without a barrier.
//
// The weights come as packed bits (gemm_layout.hpp) in the same k order, written by conv_taps_prepare below in its
// one pass over W (Sign(W), the bits, per channel tile the sums of |W| and the counts of weights that are neither
// negative nor positive); the product's set-up adds the partial sums in a fixed order into alpha = mean |W|
// (binary_weight_convolution.cpp:58-69), and its first block writes alpha and the zero count out.  Two launches per
// group make the whole forward.
//
// Numerics: q = rint(x * 2^s) with s chosen so that the slab's largest finite magnitude lands in [2^28, 2^29); the
// four digit products are accumulated exactly in int32, combined exactly in integers with the windows' sums of q
// (the bits stand for 0 / 1: sum q * (1 - 2 b) = sum q - 2 sum q b) and rounded once to fp32.  The only error is
// the rounding of x to a multiple of 2^-s: at most 2^-29 of the slab's largest magnitude per element, i.e. finer than
// fp32 itself for every window whose own largest value is within 2^-5 of the slab's.  A window that holds a NaN or an
// infinity gives NaN in all its outputs; other windows of the slab are not affected (such values are left out of the
// scale and read as 0).
#include "common.hpp"
#include "conv_geom.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kSlabThreads = 512;
constexpr int kSlabRows = 32;        // windows per block: one MFMA fragment
constexpr int kSlabDigits = 4;
constexpr int kSlabPixPad = 16;      // bytes between two pixels: consecutive pixels start 4 banks apart
constexpr int kSlabMaxTaps = 64;
constexpr int kSlabAhead = 4;        // k tiles of packed words a wavefront holds in registers ahead of its MFMAs
constexpr int kSlabTopBit = 28;      // the slab's largest magnitude lands in [2^28, 2^29): four q add up in 32 bits
constexpr int kSlabReduceBytes = 8 * 16 * 64 * 4; // one fragment of one digit's accumulators from each wavefront
constexpr int kSlabLdsLimit = 156 * 1024;
constexpr int kPrepThreads = 256;

// Sizes and LDS offsets of one launch (host and device).
struct SlabPlan {
  int tile_rows, tiles_per_sample, wide_groups;
  int ct;          // channel tiles of 32 (channels padded)
  int frags;       // fragments of 32 output channels
  int pix_stride;  // bytes per pixel: 128 per channel tile, and the padding
  int cap;         // pixels a slab may hold (the zero pixel not counted)
  int slab_bytes;
  int k_tiles;     // taps * ct
  int pixsum_off, rowsum_off, pixbad_off, rowpix_off, rowidx_off, rowbad_off, alpha_off, misc_off, total;
  // the prepared weights of one group: packed bits [k tile][wide group][lane], partial |W| sums [ct][frags * 32],
  // partial zero counts [ct][wide groups * 32]
  size_t bits_bytes, wsum_off, zeros_off, prep_bytes;
};

struct ConvSlabArgs {
  const float *x;
  const uint4_t *bits;
  const float *wsum;  // null: no alpha (BinaryConnect)
  const int *zeros;
  float *alpha_out;   // may be null
  int *zero_count;    // may be null
  const float *bias;
  const float *in_scale; // may be null: input channel c of the group is multiplied by in_scale[c] first
  const float *redo_w;   // may be null: Sign(W) of the group [Og, Cg * taps]; windows holding a NaN or an infinity are
                         // then recomputed element by element (else all their outputs are NaN)
  float *y;
  int accumulate;        // add to y instead of overwriting it
  ConvGeom g;
  int grp;
  float inv_k;
  SlabPlan p;
};

// Flattened input offset of output position p's window origin (may be negative).
inline int64_t slab_origin(const ConvGeom &g, int64_t p) {
  const int o2 = (int)(p % g.out_sp[2]);
  p /= g.out_sp[2];
  const int o1 = (int)(p % g.out_sp[1]);
  const int o0 = (int)(p / g.out_sp[1]);
  const int64_t b0 = (int64_t)o0 * g.stride[0] - g.pad[0], b1 = (int64_t)o1 * g.stride[1] - g.pad[1],
                b2 = (int64_t)o2 * g.stride[2] - g.pad[2];
  return (b0 * g.in_sp[1] + b1) * g.in_sp[2] + b2;
}
__host__ __device__ inline int64_t slab_last_tap(const ConvGeom &g) {
  return (((int64_t)(g.k[0] - 1) * g.dil[0]) * g.in_sp[1] + (int64_t)(g.k[1] - 1) * g.dil[1]) * g.in_sp[2] +
         (int64_t)(g.k[2] - 1) * g.dil[2];
}

__global__ __launch_bounds__(kSlabThreads, 1) void binary_conv_slab_kernel(ConvSlabArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const ConvGeom &g = a.g;
  const SlabPlan &P = a.p;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Blocks go to the eight XCDs round-robin: an XCD takes a contiguous run of tiles, so the tiles of one sample --
  // whose slabs overlap and whose outputs share cache lines -- meet in one L2.
  const int64_t work = xcd_remap(blockIdx.x, gridDim.x);
  const int wg = (int)(work % P.wide_groups);
  const int tile_all = (int)(work / P.wide_groups);
  const int n = tile_all / P.tiles_per_sample, tile = tile_all - n * P.tiles_per_sample;
  const int p0 = tile * P.tile_rows;
  const int rows = min(P.tile_rows, (int)g.out_sp_size - p0);
  const int taps = (int)g.k_size, plane = (int)g.in_sp_size, Cg = (int)g.Cg, CT = P.ct;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2];

  long long *s_pixsum = reinterpret_cast<long long *>(smem + P.pixsum_off);
  long long *s_rowsum = reinterpret_cast<long long *>(smem + P.rowsum_off);
  uint32_t *s_pixbad = reinterpret_cast<uint32_t *>(smem + P.pixbad_off);
  uint32_t *s_rowpix = reinterpret_cast<uint32_t *>(smem + P.rowpix_off); // [tap][row]: byte offset inside a plane
  uint32_t *s_rowidx = reinterpret_cast<uint32_t *>(smem + P.rowidx_off); // [tap][row]: pixel index
  int *s_rowbad = reinterpret_cast<int *>(smem + P.rowbad_off);
  float *s_alpha = reinterpret_cast<float *>(smem + P.alpha_off), *s_bias = s_alpha + kWideGroup;
  int *s_misc = reinterpret_cast<int *>(smem + P.misc_off); // the wavefronts' maxima

  // ---- 0. the block's rows and the slab's extent.  Every wavefront holds all 32 rows (lane % 32), so each finds the
  // extent by itself and can start loading the slab before anything goes through LDS.
  const int r = lane & 31, half = lane >> 5;
  const bool row_in = r < rows;
  int b0, b1, b2, origin;
  {
    int p = row_in ? p0 + r : p0; // rows past the tile repeat its first row
    const int o2 = p % g.out_sp[2];
    p /= g.out_sp[2];
    const int o1 = p % g.out_sp[1];
    const int o0 = p / g.out_sp[1];
    b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
    origin = (b0 * in1 + b1) * in2 + b2;
  }
  int lo, npix;
  {
    int omin = origin, omax = origin;
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) {
      omin = min(omin, __shfl_xor(omin, off));
      omax = max(omax, __shfl_xor(omax, off));
    }
    omin = __builtin_amdgcn_readfirstlane(omin), omax = __builtin_amdgcn_readfirstlane(omax);
    lo = min(max(omin, 0), plane - 1);
    const int hi = min(max(omax + (int)slab_last_tap(g), 0), plane - 1);
    npix = min(hi - lo + 1, P.cap); // (the host sized the LDS for the exact maximum: the clamp never acts)
  }
  // ---- 1. the slab: largest finite magnitude, then the digits.  A work item is 64 pixels x 16 channels (lanes along
  // the pixels, sixteen loads per lane); wavefront w takes items w, w + 8, ...  A slab of at most two items per
  // wavefront (64 pixels x 256 channels, say) is loaded once, all loads in flight together, and kept in registers
  // between the two steps; a larger one is read twice.
  const float *xs = a.x + ((int64_t)n * g.C + (int64_t)a.grp * g.Cg) * plane + lo;
  const int groups16 = 2 * CT, items = ((npix + 63) >> 6) * groups16;
  // item -> (first pixel, first channel)
  auto item_of = [&](int item, int &pix0, int &ch0) __attribute__((always_inline)) {
    const int pc = item / groups16;
    pix0 = pc * 64, ch0 = (item - pc * groups16) * 16;
  };
  auto load_item = [&](int item, float (&v)[16]) __attribute__((always_inline)) {
    int pix0, ch0;
    item_of(item < items ? item : 0, pix0, ch0);
    const int pix = pix0 + lane;
    const float *src = xs + (pix < npix ? pix : 0);
#pragma unroll
    for (int c = 0; c < 16; ++c)
      v[c] = (item < items && ch0 + c < Cg) ? src[(int64_t)(ch0 + c) * plane] : 0.0f;
    if (a.in_scale) { // one rounded product per element, before anything else
#pragma unroll
      for (int c = 0; c < 16; ++c)
        v[c] = v[c] * ((item < items && ch0 + c < Cg) ? a.in_scale[ch0 + c] : 0.0f);
    }
  };
  uint32_t amax = 0u;
  auto scan_item = [&](const float (&v)[16]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const uint32_t m = __float_as_uint(v[c]) & 0x7fffffffu;
      amax = max(amax, m < 0x7f800000u ? m : 0u);
    }
  };
  int shift = 0;
  // the item's digits -> LDS: sixteen consecutive channels of a pixel are sixteen consecutive bytes of each digit
  auto convert_item = [&](int item, const float (&v)[16]) __attribute__((always_inline)) {
    uint32_t w[kSlabDigits][4];
    long long psum = 0;
    bool bad = false;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      uint32_t d[4];
      int part = 0; // four |q| < 2^29
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bool fin = (__float_as_uint(v[4 * u + c]) & 0x7fffffffu) < 0x7f800000u;
        bad = bad || !fin;
        const int q = fin ? (int)rintf(ldexpf(v[4 * u + c], shift)) : 0;
        part += q;
        // bytes: lowest digit .. top digit (the carries of the balanced form run through the addition)
        d[c] = ((uint32_t)q + 0x808080u) ^ 0x808080u;
      }
      const uint32_t t01 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u); // d0.b0 d1.b0 d0.b1 d1.b1
      const uint32_t t23 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
      const uint32_t u01 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u); // d0.b2 d1.b2 d0.b3 d1.b3
      const uint32_t u23 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
      w[3][u] = __builtin_amdgcn_perm(t23, t01, 0x05040100u); // lowest digits of the four channels
      w[2][u] = __builtin_amdgcn_perm(t23, t01, 0x07060302u);
      w[1][u] = __builtin_amdgcn_perm(u23, u01, 0x05040100u);
      w[0][u] = __builtin_amdgcn_perm(u23, u01, 0x07060302u); // top digits
      psum += part;
    }
    int pix0, ch0;
    item_of(item < items ? item : 0, pix0, ch0);
    if (item < items && pix0 + lane < npix) {
      // channel tile ch0 / 32, half (ch0 / 16) % 2 of its 32 channels: one byte per channel and digit
      unsigned char *dst = smem + (pix0 + lane + 1) * P.pix_stride + (ch0 >> 5) * 128 + (ch0 & 16);
#pragma unroll
      for (int dg = 0; dg < kSlabDigits; ++dg) {
        uint4_t o;
        o.x = w[dg][0], o.y = w[dg][1], o.z = w[dg][2], o.w = w[dg][3];
        *reinterpret_cast<uint4_t *>(dst + dg * 32) = o;
      }
      if (psum != 0)
        atomicAdd(reinterpret_cast<unsigned long long *>(&s_pixsum[pix0 + lane + 1]), (unsigned long long)psum);
      if (bad)
        s_pixbad[pix0 + lane + 1] = 1u;
    }
  };
  const bool hold = items <= 16; // uniform over the block
  float hv[2][16];
  if (hold) {
    load_item(wave, hv[0]);
    load_item(wave + 8, hv[1]);
  }
  // the partial |W| sums of the block's channels (the first eight channel tiles) and the bias: used in the epilogue
  float av[8], bias_v = -0.0f;
  const int ogp = P.frags * 32, col = wg * kWideGroup + (tid & (kWideGroup - 1));
  if (tid < kWideGroup) {
    if (a.wsum) {
      const float *part = a.wsum + (col < ogp ? col : ogp - 1);
#pragma unroll
      for (int c = 0; c < 8; ++c)
        av[c] = part[(int64_t)(c < CT ? c : CT - 1) * ogp];
    }
    if (a.bias)
      bias_v = a.bias[col < g.Og ? col : g.Og - 1];
  }
  // while the loads are in flight: the tables in LDS
  for (int i = tid; i <= P.cap; i += kSlabThreads) {
    s_pixsum[i] = 0;
    s_pixbad[i] = 0u;
  }
  if (tid < kSlabRows) {
    s_rowsum[tid] = 0;
    s_rowbad[tid] = 0;
    s_rowpix[taps * kSlabRows + tid] = 0u; // the entry of steps past the last k tile: the zero pixel
  }
  for (int i = tid; i < (P.pix_stride >> 2); i += kSlabThreads) // the zero pixel
    *reinterpret_cast<uint32_t *>(smem + 4 * i) = 0u;
  for (int t = tid >> 5; t < taps; t += kSlabThreads / 32) { // tap t of row r: its pixel in the slab, if any
    int q = t;
    const int k2 = q % g.k[2];
    q /= g.k[2];
    const int k1 = q % g.k[1], k0 = q / g.k[1];
    const int e0 = k0 * g.dil[0], e1 = k1 * g.dil[1], e2 = k2 * g.dil[2];
    const int i0 = b0 + e0, i1 = b1 + e1, i2 = b2 + e2;
    const bool ok = row_in && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                    (unsigned)i2 < (unsigned)in2;
    const int idx = origin + (e0 * in1 + e1) * in2 + e2 - lo + 1;
    const bool held = ok && idx >= 1 && idx <= npix;
    s_rowidx[t * kSlabRows + r] = held ? (uint32_t)idx : 0u;
    s_rowpix[t * kSlabRows + r] = held ? (uint32_t)(idx * P.pix_stride) : 0u;
  }
  if (hold) {
    scan_item(hv[0]);
    scan_item(hv[1]);
  } else {
    for (int item = wave; item < items; item += 8) {
      float v[16];
      load_item(item, v);
      scan_item(v);
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    amax = max(amax, (uint32_t)__shfl_xor((int)amax, off));
  if (lane == 0)
    s_misc[wave] = (int)amax;
  __syncthreads();
  {
    uint32_t bmax = 0u;
#pragma unroll
    for (int w = 0; w < 8; ++w)
      bmax = max(bmax, (uint32_t)s_misc[w]);
    if (bmax != 0u)
      shift = kSlabTopBit - binade_exponent(binade_of(bmax));
  }
  if (hold) {
    convert_item(wave, hv[0]);
    convert_item(wave + 8, hv[1]);
  } else {
    for (int item = wave; item < items; item += 8) {
      float v[16];
      load_item(item, v);
      convert_item(item, v);
    }
  }
  if (tid < kWideGroup) { // alpha = (sum of the partial sums, in channel-tile order: every block forms the same bits) / K
    float al = 1.0f;
    if (a.wsum) {
      float acc = 0.0f;
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if (c < CT)
          acc += av[c];
      for (int c = 8; c < CT; ++c)
        acc += a.wsum[(int64_t)c * ogp + (col < ogp ? col : ogp - 1)];
      al = acc * a.inv_k;
      if (tile_all == 0 && a.alpha_out && col < g.Og)
        a.alpha_out[col] = al;
    }
    s_alpha[tid] = al;
    s_bias[tid] = bias_v;
  }
  if (work == 0 && wave == 7 && a.zero_count) {
    int z = 0;
    for (int i = lane; i < CT * P.wide_groups * 32; i += 64)
      z += a.zeros[i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      z += __shfl_xor(z, off);
    if (lane == 0)
      *a.zero_count = z;
  }
  __syncthreads();
  // the windows' sums of q and whether they hold a non-finite value (read again only after the product)
  {
    long long sum = 0;
    uint32_t bad = 0u;
    for (int t = tid >> 5; t < taps; t += kSlabThreads / 32) {
      const uint32_t idx = s_rowidx[t * kSlabRows + r];
      sum += s_pixsum[idx];
      bad |= s_pixbad[idx];
    }
    if (sum != 0)
      atomicAdd(reinterpret_cast<unsigned long long *>(&s_rowsum[r]), (unsigned long long)sum);
    if (bad)
      s_rowbad[r] = 1;
  }

  // ---- 2. the product.  Wavefront (wn, wk): channel fragments 2 wn, 2 wn + 1 of the wide group, k tiles wk, wk + 2, ...
  const int wn = wave & 3, wk = wave >> 2;
  const int nk = (P.k_tiles - wk + 1) / 2;
  i32x16_t acc[kSlabDigits][2];
#pragma unroll
  for (int d = 0; d < kSlabDigits; ++d)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        acc[d][j][q] = 0;
  uint32_t frag_mask[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    frag_mask[j] = 0x01010101u << (2 * wn + j);
    asm volatile("" : "+s"(frag_mask[j]));
  }
  if (nk > 0) {
    // the words of step i sit at wnext[lane] when they are loaded: a uniform pointer that stops at the last step
    const uint4_t *wnext = a.bits + ((int64_t)wk * P.wide_groups + wg) * 64;
    const int64_t wstep = (int64_t)2 * P.wide_groups * 64;
    int wleft = nk - 1; // steps the pointer may still advance
    uint4_t words[kSlabAhead];
#pragma unroll
    for (int u = 0; u < kSlabAhead; ++u) {
      words[u] = wnext[lane];
      wnext += wleft > 0 ? wstep : 0;
      --wleft;
    }
    // position (tap, channel tile) of the k tile two steps ahead, advanced by two k tiles per step
    int tap2 = 0, ct2 = wk;
    auto normalise = [&]() __attribute__((always_inline)) {
      if (ct2 >= CT) {
        ct2 -= CT, ++tap2;
        if (ct2 >= CT)
          ct2 -= CT, ++tap2;
      }
    };
    normalise();
    const uint32_t lane_off = (uint32_t)(half * 16);
    const uint32_t *my_rowpix = s_rowpix + r;
    // LDS offset of the lane's sixteen bytes of step (tap2, ct2); past the last k tile: inside the zero pixel
    auto row_off = [&]() __attribute__((always_inline)) {
      return my_rowpix[(tap2 < taps ? tap2 : taps) * kSlabRows] + (uint32_t)(ct2 * 128) + lane_off;
    };
    auto advance = [&]() __attribute__((always_inline)) {
      ct2 += 2;
      normalise();
    };
    auto read_a = [&](uint32_t off, uint4_t (&af)[kSlabDigits]) __attribute__((always_inline)) {
#pragma unroll
      for (int d = 0; d < kSlabDigits; ++d)
        af[d] = *reinterpret_cast<const uint4_t *>(smem + off + d * 32);
    };
    // bits -> bytes in {0, 2^F}: register i of channel fragment F is word_i & (0x01010101 << F)
    auto mma = [&](const uint4_t (&af)[kSlabDigits], const uint4_t &w) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        uint4_t bf;
        bf.x = w.x & frag_mask[j], bf.y = w.y & frag_mask[j], bf.z = w.z & frag_mask[j], bf.w = w.w & frag_mask[j];
#pragma unroll
        for (int d = 0; d < kSlabDigits; ++d)
          acc[d][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, bf),
                                                            __builtin_bit_cast(i32x4_t, af[d]), acc[d][j], 0, 0, 0);
      }
    };
    uint32_t off_a = row_off(); // step 0
    advance();
    uint32_t off_b = row_off(); // step 1
    advance();
    uint4_t af[2][kSlabDigits];
    read_a(off_a, af[0]);
    // Whole rounds of kSlabAhead steps, without a branch inside a round (the compiler then counts the loads in flight
    // exactly: a word is waited for with the younger loads still outstanding).  Steps past the last k tile
    // multiply the zero pixel.  Inside a step the LDS reads of the next step (the table entry and the four digits) and
    // the load of a later step's words are dealt out one per MFMA of this step (sched_group_barrier: 0x008 = MFMA,
    // 0x100 = LDS read, 0x020 = global load): a wavefront that issues them in a row leaves the matrix pipe waiting.
    for (int i0 = 0; i0 < nk; i0 += kSlabAhead) {
#pragma unroll
      for (int u = 0; u < kSlabAhead; ++u) {
        const uint32_t off_c = row_off(); // step i + 2
        advance();
        read_a(off_b, af[(u + 1) & 1]); // step i + 1
        mma(af[u & 1], words[u]);
        words[u] = wnext[lane];
        wnext += wleft > 0 ? wstep : 0;
        --wleft;
#pragma unroll
        for (int q = 0; q < kSlabDigits + 1; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, kSlabDigits - 2, 0);
        __builtin_amdgcn_sched_barrier(0);
        off_b = off_c;
      }
    }
  }

  // ---- 3. the two k groups' accumulators added exactly through LDS (the planes are free once every wavefront has
  // left the loop), one digit at a time, in two alternating areas: wavefront (wn, wk) hands the fragment it does not
  // finish (1 - wk) to its partner (wn, 1 - wk) and adds the partner's copy of fragment wk to its own.
  i32x16_t fin[kSlabDigits];
  {
    uint4_t *red = reinterpret_cast<uint4_t *>(smem);
    const int mine = wave * 4 * 64 + lane, theirs = (wave ^ 4) * 4 * 64 + lane;
    __syncthreads();
#pragma unroll
    for (int d = 0; d < kSlabDigits; ++d) {
      uint4_t *area = red + (d & 1) * (kSlabReduceBytes / 16);
      const i32x16_t give = wk ? acc[d][0] : acc[d][1];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint4_t v;
        v.x = give[4 * q + 0], v.y = give[4 * q + 1], v.z = give[4 * q + 2], v.w = give[4 * q + 3];
        area[mine + q * 64] = v;
      }
      __syncthreads();
      fin[d] = wk ? acc[d][1] : acc[d][0];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4_t v = area[theirs + q * 64];
        fin[d][4 * q + 0] += (int)v.x, fin[d][4 * q + 1] += (int)v.y;
        fin[d][4 * q + 2] += (int)v.z, fin[d][4 * q + 3] += (int)v.w;
      }
    }
  }

  // ---- 4. epilogue.  Accumulator register q of lane l: channel 8 (q / 4) + 4 (l / 32) + q % 4 of the fragment,
  // window l % 32.  dot = rowsum - 2 * sum(q * bit); the accumulators carry the factor 2^F of the fragment's byte
  // (-128 for F = 7).  With m_d = acc_d / 2^F:  sum(q * bit) = hi * 2^16 + lo, hi = m_0 * 256 + m_1,
  // lo = m_2 * 256 + m_3 (|m_d| <= 2^21 for the k the host admits), and with rowsum = s_hi * 2^16 + s_lo the result is
  // (s_hi -+ 2 hi) * 2^16 + (s_lo -+ 2 lo) = A * 2^16 + B with 0 <= B < 2^16: one fused multiply-add, rounded once
  // while |A| < 2^24 (sums below 2^40), else twice (2^-24 of the sum).
  if (!row_in)
    return;
  const long long rowsum = s_rowsum[r];
  const bool rowbad = s_rowbad[r] != 0;
  const int s_hi = (int)(rowsum >> 16), s_lo = (int)(rowsum & 0xffff);
  const int F = 2 * wn + wk;
  const bool negate = F == 7;
  // channel of register q: c0 + 8 (q / 4) + q % 4; everything an output needs besides its accumulators is fetched
  // before the stores (the compiler does not move a load across them)
  const int c0 = F * 32 + 4 * half, og_left = (int)g.Og - wg * kWideGroup - c0; // channels from c0 to the group's last
  const int osz = (int)g.out_sp_size;
  float al[16], bi[16];
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    al[q] = s_alpha[c0 + 8 * (q >> 2) + (q & 3)];
    bi[q] = s_bias[c0 + 8 * (q >> 2) + (q & 3)];
  }
  float *ybase = a.y + (((int64_t)n * g.O + (int64_t)a.grp * g.Og + (int64_t)wg * kWideGroup + c0) * g.out_sp_size + p0 + r);
  float prev[16];
  if (a.accumulate) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int cq = 8 * (q >> 2) + (q & 3);
      prev[q] = cq < og_left ? ybase[cq * osz] : 0.0f;
    }
  }
  const float bad_scale = rowbad ? __uint_as_float(0x7fc00000u) : 65536.0f; // NaN through the multiply-add
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int cq = 8 * (q >> 2) + (q & 3);
    const int hi = ((fin[0][q] >> F) << 8) + (fin[1][q] >> F), lo = ((fin[2][q] >> F) << 8) + (fin[3][q] >> F);
    int A = negate ? s_hi + 2 * hi : s_hi - 2 * hi, B = negate ? s_lo + 2 * lo : s_lo - 2 * lo;
    A += B >> 16, B &= 0xffff; // the sum is A * 2^16 + B, 0 <= B < 2^16
    float v = ldexpf(fmaf((float)A, bad_scale, (float)B), -shift);
    if (a.accumulate)
      v = prev[q] + v;
    v = v * al[q];
    v = v + bi[q];
    if (cq < og_left)
      ybase[cq * osz] = v; // (Og * out_sp_size < 2^31: checked by the host)
  }
  // A window holding a NaN or an infinity (rare): the reference's product propagates such values output by output
  // (convolution.cpp:185-193: the row of the unfolded input, zeros where the window leaves the input, times
  // Ws = Wb * alpha, then + b: Inf * w = +-Inf, Inf - Inf = NaN), so the lane recomputes its sixteen outputs as plain
  // fp32 dot products over the materialised signs and replaces the NaN stored above.
  if (rowbad && a.redo_w) {
    int p = p0 + r;
    const int o2 = p % g.out_sp[2];
    p /= g.out_sp[2];
    const int o1 = p % g.out_sp[1], o0 = p / g.out_sp[1];
    const int w0 = o0 * g.stride[0] - g.pad[0], w1 = o1 * g.stride[1] - g.pad[1], w2 = o2 * g.stride[2] - g.pad[2];
    const float *xn = a.x + ((int64_t)n * g.C + (int64_t)a.grp * g.Cg) * plane;
#pragma unroll 1
    for (int q = 0; q < 16; ++q) {
      const int cq = 8 * (q >> 2) + (q & 3);
      if (cq >= og_left)
        continue;
      const float *wrow = a.redo_w + ((int64_t)wg * kWideGroup + c0 + cq) * ((int64_t)Cg * taps);
      const float scale = s_alpha[c0 + cq];
      float acc = 0.0f;
#pragma unroll 1
      for (int c = 0; c < Cg; ++c) {
        int t = 0;
        for (int k0 = 0; k0 < g.k[0]; ++k0)
          for (int k1 = 0; k1 < g.k[1]; ++k1)
            for (int k2 = 0; k2 < g.k[2]; ++k2, ++t) {
              const int i0 = w0 + k0 * g.dil[0], i1 = w1 + k1 * g.dil[1], i2 = w2 + k2 * g.dil[2];
              const bool in = i0 >= 0 && i0 < in0 && i1 >= 0 && i1 < in1 && i2 >= 0 && i2 < in2;
              const float xv = in ? xn[(int64_t)c * plane + (i0 * in1 + i1) * in2 + i2] : 0.0f;
              acc = acc + xv * (wrow[c * taps + t] * scale);
            }
      }
      ybase[cq * osz] = acc + s_bias[c0 + cq];
    }
  }
#endif
}

// One pass over the weights W [Og, Cg, taps] of a group: Wb = Sign(W) (sign.hpp:48-50), the packed bits of the product
// above in the order k' = tap * (32 ct) + channel, and per channel tile the sums of |W| and the counts of weights that
// are neither negative nor positive.  Block (wide group, channel tile ct, r): the eight output channels
// 256 wg + 32 F + r, F = 0..7 -- the ones whose bits share the packed words of lanes r and r + 32 -- and the 32 input
// channels of the tile: a contiguous run of 32 * taps floats per row.  The signs go to LDS as bytes, from where
// thread (tap, half) assembles its packed word; |w| goes through LDS so that a row's sum is formed by one wavefront in
// a fixed order.
__global__ __launch_bounds__(kPrepThreads) void conv_taps_prepare(const float *__restrict__ W, float *__restrict__ Wb,
                                                                  uint4_t *__restrict__ bits, float *__restrict__ wsum,
                                                                  int *__restrict__ zeros, int Og, int Cg, int taps,
                                                                  int ct_count, int frags, int wide_groups,
                                                                  float zero_to) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // [8 rows][32 * taps]: |w| as floats, then the "negative" flags as bytes
  const int seg_full = 32 * taps;
  float *s_abs = reinterpret_cast<float *>(smem);
  unsigned char *s_neg = smem + (size_t)8 * seg_full * 4;
  __shared__ int s_zero[kPrepThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x / 32, r = blockIdx.x % 32, ct = blockIdx.y;
  const int c0 = ct * 32, cn = min(32, Cg - c0), seg = cn * taps, elems = 8 * seg;
  const int64_t Kg = (int64_t)Cg * taps;
  for (int i = tid; i < 8 * seg_full / 4; i += kPrepThreads)
    reinterpret_cast<uint32_t *>(s_neg)[i] = 0u; // rows and channels past the end: bit clear (their digits are 0)
  __syncthreads();
  int nzero = 0;
  for (int base = 0; base < elems; base += 12 * kPrepThreads) {
    float w[12];
    int64_t at[12];
#pragma unroll
    for (int m = 0; m < 12; ++m) {
      const int idx = base + tid + kPrepThreads * m;
      const int f = idx / seg, kl = idx - f * seg;
      const int n = wg * kWideGroup + 32 * f + r;
      const bool in = idx < elems && n < Og;
      at[m] = in ? (int64_t)n * Kg + (int64_t)c0 * taps + kl : -1;
      w[m] = in ? W[at[m]] : 1.0f;
    }
#pragma unroll
    for (int m = 0; m < 12; ++m) {
      const int idx = base + tid + kPrepThreads * m;
      const int f = idx / seg, kl = idx - f * seg;
      if (idx < elems)
        s_abs[f * seg_full + kl] = at[m] >= 0 ? fabsf(w[m]) : 0.0f;
      if (at[m] >= 0) {
        const bool is_zero = !(w[m] > 0.0f) && !(w[m] < 0.0f);
        const bool neg = (w[m] < 0.0f) || (is_zero && zero_to < 0.0f);
        if (Wb)
          Wb[at[m]] = (w[m] > 0.0f) ? 1.0f : ((w[m] < 0.0f) ? -1.0f : zero_to);
        s_neg[f * seg_full + kl] = neg ? 1 : 0;
        nzero += is_zero ? 1 : 0;
      }
    }
  }
  __syncthreads();
  for (int f = wave; f < 8; f += kPrepThreads / 64) {
    float asum = 0.0f;
    for (int kl = lane; kl < seg; kl += 64)
      asum += s_abs[f * seg_full + kl];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      asum += __shfl_xor(asum, off);
    const int n = wg * kWideGroup + 32 * f + r;
    if (lane == 0 && n < frags * 32)
      wsum[(int64_t)ct * frags * 32 + n] = asum; // rows past Og: zero
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    nzero += __shfl_xor(nzero, off);
  if (lane == 0)
    s_zero[wave] = nzero;
  __syncthreads();
  if (tid == 0)
    zeros[(ct * wide_groups + wg) * 32 + r] = s_zero[0] + s_zero[1] + s_zero[2] + s_zero[3];
  // the packed words of lanes r and r + 32 of the block's k tiles (tap, ct): word i, byte c, bit F <- row F, channel
  // c0 + 16 half + 4 i + c
  for (int item = tid; item < 2 * taps; item += kPrepThreads) {
    const int t = item >> 1, g16 = item & 1;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const unsigned char *src = s_neg + f * seg_full + (g16 * 16) * taps + t;
#pragma unroll
      for (int j = 0; j < 16; ++j)
        o[j >> 2] |= (uint32_t)src[j * taps] << (8 * (j & 3) + f);
    }
    uint4_t v;
    v.x = o[0], v.y = o[1], v.z = o[2], v.w = o[3];
    bits[((int64_t)(t * ct_count + ct) * wide_groups + wg) * 64 + g16 * 32 + r] = v;
  }
}

// The packed bits of the same product run backwards, for the gradient with respect to the input of a convolution of
// unit stride: dx = conv(dy, W') with W'[c][o][t] = Sign(W)[o][c][taps - 1 - t] and the padding (k - 1) dil - pad
// (convolution.cpp:199-283 unfolds dy . W^T and folds it back; here the fold is the contraction over the taps).
// Block (wide group of input channels c, tile of 32 output channels o, r) as in conv_taps_prepare; only the bits are
// written.
__global__ __launch_bounds__(kPrepThreads) void conv_taps_prepare_transposed(const float *__restrict__ W,
                                                                             uint4_t *__restrict__ bits, int Og, int Cg,
                                                                             int taps, int ct_count, int wide_groups,
                                                                             float zero_to) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int seg_full = 32 * taps;
  unsigned char *s_neg = smem; // [8 rows c][32 channels o][tap, flipped]
  const int tid = threadIdx.x;
  const int wg = blockIdx.x / 32, r = blockIdx.x % 32, ct = blockIdx.y;
  const int o0 = ct * 32;
  for (int idx = tid; idx < 8 * seg_full; idx += kPrepThreads) {
    const int f = idx / seg_full, rem = idx - f * seg_full, ol = rem / taps, t = rem - ol * taps;
    const int c = wg * kWideGroup + 32 * f + r, o = o0 + ol;
    unsigned char neg = 0;
    if (c < Cg && o < Og) {
      const float w = W[((int64_t)o * Cg + c) * taps + t];
      const bool is_zero = !(w > 0.0f) && !(w < 0.0f);
      neg = ((w < 0.0f) || (is_zero && zero_to < 0.0f)) ? 1 : 0;
    }
    s_neg[f * seg_full + ol * taps + (taps - 1 - t)] = neg;
  }
  __syncthreads();
  for (int item = tid; item < 2 * taps; item += kPrepThreads) {
    const int t = item >> 1, g16 = item & 1;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int f = 0; f < 8; ++f) {
      const unsigned char *src = s_neg + f * seg_full + (g16 * 16) * taps + t;
#pragma unroll
      for (int j = 0; j < 16; ++j)
        o[j >> 2] |= (uint32_t)src[j * taps] << (8 * (j & 3) + f);
    }
    uint4_t v;
    v.x = o[0], v.y = o[1], v.z = o[2], v.w = o[3];
    bits[((int64_t)(t * ct_count + ct) * wide_groups + wg) * 64 + g16 * 32 + r] = v;
  }
}

// The largest run of input positions a tile's windows span: a window's first position grows along an output row, so
// a tile's lowest origin is at its first position or at the start of a row inside it, its highest at its last
// position or at the end of a row inside it.
int64_t slab_longest_run(const ConvGeom &g, int tile_rows, int tiles_per_sample) {
  const int64_t plane = g.in_sp_size, last = slab_last_tap(g), ow = g.out_sp[2];
  int64_t longest = 1;
  for (int64_t t = 0; t < tiles_per_sample; ++t) {
    const int64_t p0 = t * tile_rows, p1 = (p0 + tile_rows < g.out_sp_size ? p0 + tile_rows : g.out_sp_size) - 1;
    int64_t omin = slab_origin(g, p0), omax = slab_origin(g, p1);
    if (omin > omax) {
      const int64_t s = omin;
      omin = omax, omax = s;
    }
    for (int64_t row = p0 / ow + 1; row * ow <= p1; ++row) {
      const int64_t first = slab_origin(g, row * ow), prev = slab_origin(g, row * ow - 1);
      omin = first < omin ? first : omin, omax = first > omax ? first : omax;
      omin = prev < omin ? prev : omin, omax = prev > omax ? prev : omax;
    }
    const int64_t lo = omin < 0 ? 0 : (omin > plane - 1 ? plane - 1 : omin);
    const int64_t hi_raw = omax + last, hi = hi_raw < 0 ? 0 : (hi_raw > plane - 1 ? plane - 1 : hi_raw);
    if (hi - lo + 1 > longest)
      longest = hi - lo + 1;
  }
  return longest;
}

bool compute_slab_plan(const ConvGeom &g, SlabPlan &p);

// The plan of a geometry is asked for several times per call (does it apply, how much workspace, the launches) and
// sizing the slab walks the tiles of a sample: the last few answers are kept per thread.
bool make_slab_plan(const ConvGeom &g, SlabPlan &p) {
  struct Key {
    int64_t outer, C, O, group;
    int in_sp[kMaxSpatial], k[kMaxSpatial], pad[kMaxSpatial], stride[kMaxSpatial], dil[kMaxSpatial];
    bool operator==(const Key &o) const {
      bool same = outer == o.outer && C == o.C && O == o.O && group == o.group;
      for (int i = 0; i < kMaxSpatial; ++i)
        same = same && in_sp[i] == o.in_sp[i] && k[i] == o.k[i] && pad[i] == o.pad[i] && stride[i] == o.stride[i] &&
               dil[i] == o.dil[i];
      return same;
    }
  };
  constexpr int kKept = 4; // a forward and a backward geometry alternate in training
  static thread_local bool have[kKept] = {false, false, false, false}, kept_ok[kKept];
  static thread_local Key kept_key[kKept];
  static thread_local SlabPlan kept_plan[kKept];
  static thread_local int next = 0;
  Key key;
  key.outer = g.outer, key.C = g.C, key.O = g.O, key.group = g.group;
  for (int i = 0; i < kMaxSpatial; ++i)
    key.in_sp[i] = g.in_sp[i], key.k[i] = g.k[i], key.pad[i] = g.pad[i], key.stride[i] = g.stride[i],
    key.dil[i] = g.dil[i];
  for (int e = 0; e < kKept; ++e)
    if (have[e] && key == kept_key[e]) {
      p = kept_plan[e];
      return kept_ok[e];
    }
  const int e = next;
  next = (next + 1) % kKept;
  kept_ok[e] = compute_slab_plan(g, kept_plan[e]);
  kept_key[e] = key;
  have[e] = true;
  p = kept_plan[e];
  return kept_ok[e];
}

bool compute_slab_plan(const ConvGeom &g, SlabPlan &p) {
  if (g.k_size > kSlabMaxTaps || g.Cg < 24 || g.in_sp_size >= ((int64_t)1 << 30) ||
      g.out_sp_size >= ((int64_t)1 << 30) || g.Og >= ((int64_t)1 << 24) ||
      (g.Og + kWideGroup) * g.out_sp_size >= ((int64_t)1 << 31))
    return false;
  const int64_t cgp = ceil_div(g.Cg, 32) * 32;
  // padded channels cost as much as real ones; the epilogue's 32-bit steps hold kChunkK terms
  if (cgp * 3 > g.Cg * 4 || g.k_size * cgp > kChunkK)
    return false;
  const int64_t ow = g.out_sp[2], map_rows = g.out_sp_size / ow;
  if (ow <= kSlabRows) { // whole rows of the output map, evenly
    const int64_t per = kSlabRows / ow, tiles = ceil_div(map_rows, per);
    p.tile_rows = (int)(ceil_div(map_rows, tiles) * ow);
  } else {
    p.tile_rows = (int)ceil_div(g.out_sp_size, ceil_div(g.out_sp_size, kSlabRows));
  }
  const int64_t tiles = ceil_div(g.out_sp_size, p.tile_rows);
  if (tiles > 16384) // the host walks them to size the slab
    return false;
  p.tiles_per_sample = (int)tiles;
  p.wide_groups = (int)bits_wide_groups(g.Og);
  if (g.outer * tiles * p.wide_groups >= ((int64_t)1 << 31))
    return false;
  p.ct = (int)(cgp / 32);
  p.frags = (int)ceil_div(g.Og, 32);
  p.pix_stride = kSlabDigits * (int)cgp + kSlabPixPad;
  const int64_t cap = slab_longest_run(g, p.tile_rows, p.tiles_per_sample);
  const int64_t slab_bytes = (cap + 1) * p.pix_stride;
  if (slab_bytes > kSlabLdsLimit)
    return false;
  p.cap = (int)cap;
  p.slab_bytes = (int)slab_bytes;
  p.k_tiles = (int)(g.k_size * p.ct);
  int64_t off = slab_bytes;
  if (off < 2 * kSlabReduceBytes) // two areas for the exchange between the k groups
    off = 2 * kSlabReduceBytes;
  p.pixsum_off = (int)off, off += 8 * (cap + 1);
  p.rowsum_off = (int)off, off += 8 * kSlabRows;
  off = (int64_t)round_up((size_t)off, 16);
  p.pixbad_off = (int)off, off += 4 * (cap + 1);
  p.rowpix_off = (int)off, off += 4 * kSlabRows * (g.k_size + 1);
  p.rowidx_off = (int)off, off += 4 * kSlabRows * g.k_size;
  p.rowbad_off = (int)off, off += 4 * kSlabRows;
  p.alpha_off = (int)off, off += 2 * 4 * kWideGroup;
  p.misc_off = (int)off, off += 64;
  p.total = (int)off;
  p.bits_bytes = (size_t)p.k_tiles * p.wide_groups * kFragBytes;
  p.wsum_off = round_up(p.bits_bytes, 256);
  p.zeros_off = p.wsum_off + round_up((size_t)p.ct * p.frags * 32 * sizeof(float), 256);
  p.prep_bytes = p.zeros_off + round_up((size_t)p.ct * p.wide_groups * 32 * sizeof(int), 256);
  return off <= kSlabLdsLimit;
}

} // namespace

bool conv_slab_applies(const ConvGeom &g) {
  SlabPlan p;
  return make_slab_plan(g, p);
}

bool conv_slab_plan_summary(const ConvGeom &g, int32_t out[4]) {
  SlabPlan p;
  if (!make_slab_plan(g, p))
    return false;
  out[0] = p.tile_rows, out[1] = p.tiles_per_sample, out[2] = p.cap, out[3] = p.total;
  return true;
}

size_t conv_slab_prepared_bytes(const ConvGeom &g) {
  SlabPlan p;
  return make_slab_plan(g, p) ? p.prep_bytes : 0;
}

int launch_conv_slab_prepare(const float *Wg, float *Wbg, void *prepared, const ConvGeom &g, float zero_to,
                             hipStream_t stream) {
  SlabPlan p;
  if (!make_slab_plan(g, p))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "the slab convolution does not cover this geometry.");
  if (!aligned16(prepared))
    return fail(NBLA_HIP_ERR_MEMORY, "prepared-weight buffer must be 16-byte aligned.");
  const size_t lds = (size_t)8 * 32 * g.k_size * 5; // |w| as floats and the sign flags as bytes
  static std::atomic<uint64_t> configured{0};
  const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(conv_taps_prepare), 8 * 32 * kSlabMaxTaps * 5,
                                   configured, "hipFuncSetAttribute(conv_taps_prepare LDS size)");
  if (rc)
    return rc;
  char *base = static_cast<char *>(prepared);
  hipLaunchKernelGGL(conv_taps_prepare, dim3((unsigned)p.wide_groups * 32, (unsigned)p.ct), dim3(kPrepThreads), lds,
                     stream, Wg, Wbg, reinterpret_cast<uint4_t *>(base), reinterpret_cast<float *>(base + p.wsum_off),
                     reinterpret_cast<int *>(base + p.zeros_off), (int)g.Og, (int)g.Cg, (int)g.k_size, p.ct, p.frags,
                     p.wide_groups, zero_to);
  NBLA_HIP_LAUNCH_CHECK("conv_taps_prepare");
  return NBLA_HIP_OK;
}

// The convolution that computes the input gradient of `g` (unit stride): dy takes the place of x, the roles of the
// channels are exchanged, the padding becomes (k - 1) dil - pad.  False when `g` has a stride or needs a negative
// padding, or when the slab product does not cover the result.
bool conv_slab_transposed_geom(const ConvGeom &g, ConvGeom &t) {
  t = g;
  for (int i = 0; i < kMaxSpatial; ++i) {
    if (g.stride[i] != 1)
      return false;
    t.pad[i] = (g.k[i] - 1) * g.dil[i] - g.pad[i];
    if (t.pad[i] < 0)
      return false;
    t.in_sp[i] = g.out_sp[i];
    t.out_sp[i] = g.in_sp[i];
  }
  t.C = g.O, t.O = g.C, t.Cg = g.Og, t.Og = g.Cg;
  t.in_sp_size = g.out_sp_size, t.out_sp_size = g.in_sp_size;
  t.Kg = t.Cg * g.k_size;
  t.M = g.outer * t.out_sp_size;
  SlabPlan p;
  return make_slab_plan(t, p);
}

int launch_conv_slab_prepare_transposed(const float *Wg, void *prepared, const ConvGeom &g, float zero_to,
                                        hipStream_t stream) {
  ConvGeom t;
  SlabPlan p;
  if (!conv_slab_transposed_geom(g, t) || !make_slab_plan(t, p))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "the slab convolution does not cover this input gradient.");
  if (!aligned16(prepared))
    return fail(NBLA_HIP_ERR_MEMORY, "prepared-weight buffer must be 16-byte aligned.");
  const size_t lds = (size_t)8 * 32 * g.k_size;
  static std::atomic<uint64_t> configured{0};
  const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(conv_taps_prepare_transposed),
                                   8 * 32 * kSlabMaxTaps, configured,
                                   "hipFuncSetAttribute(conv_taps_prepare_transposed LDS size)");
  if (rc)
    return rc;
  hipLaunchKernelGGL(conv_taps_prepare_transposed, dim3((unsigned)p.wide_groups * 32, (unsigned)p.ct),
                     dim3(kPrepThreads), lds, stream, Wg, static_cast<uint4_t *>(prepared), (int)g.Og, (int)g.Cg,
                     (int)g.k_size, p.ct, p.wide_groups, zero_to);
  NBLA_HIP_LAUNCH_CHECK("conv_taps_prepare_transposed");
  return NBLA_HIP_OK;
}

int launch_conv_slab(const float *x, const ConvGeom &g, int64_t grp, const void *prepared, float *alpha_out,
                     int *zero_count, const float *bias, float *y, hipStream_t stream, const float *in_scale,
                     bool accumulate, const float *redo_w) {
  ConvSlabArgs a;
  if (!make_slab_plan(g, a.p))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "the slab convolution does not cover this geometry.");
  if (!aligned16(prepared))
    return fail(NBLA_HIP_ERR_MEMORY, "prepared-weight buffer must be 16-byte aligned.");
  int rc = ensure_init();
  if (rc)
    return rc;
  static std::atomic<uint64_t> configured{0};
  rc = allow_dynamic_lds(reinterpret_cast<const void *>(binary_conv_slab_kernel), kSlabLdsLimit, configured,
                         "hipFuncSetAttribute(binary_conv_slab LDS size)");
  if (rc)
    return rc;
  const char *base = static_cast<const char *>(prepared);
  a.x = x;
  a.bits = reinterpret_cast<const uint4_t *>(base);
  a.wsum = alpha_out ? reinterpret_cast<const float *>(base + a.p.wsum_off) : nullptr;
  a.zeros = reinterpret_cast<const int *>(base + a.p.zeros_off);
  a.alpha_out = alpha_out;
  a.zero_count = zero_count;
  a.bias = bias;
  a.in_scale = in_scale;
  a.redo_w = (in_scale || accumulate) ? nullptr : redo_w;
  a.accumulate = accumulate ? 1 : 0;
  a.y = y;
  a.g = g;
  a.grp = (int)grp;
  a.inv_k = (float)1 / g.Kg;
  const unsigned blocks = (unsigned)(g.outer * a.p.tiles_per_sample * a.p.wide_groups);
  hipLaunchKernelGGL(binary_conv_slab_kernel, dim3(blocks), dim3(kSlabThreads), (size_t)a.p.total, stream, a);
  NBLA_HIP_LAUNCH_CHECK("binary_conv_slab");
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
