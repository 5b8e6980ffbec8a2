// BinaryWeightConvolution / BinaryConnectConvolution forwards (channel-first, up
// to three spatial dimensions, groups): the convolution is the product
//   y'[pixel, o] = sum_k col[pixel, k] * Wb[o, k],   pixel = (sample, out position), k = (c, kernel tap)
// The unfolded activations are never materialised in fp32: they are gathered
// straight into the fragment-ordered digit operand of the bit-weight MFMA
// product, whose epilogue scatters into the [sample, O, out position] layout.
#include "common.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"
#include "conv_geom.hpp"

namespace nbla_hip {

// convolution.cpp:41-160
int make_geom(ConvGeom &g, int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O, const int64_t *kernel,
              const int64_t *pad, const int64_t *stride, const int64_t *dil, int64_t group) {
  if (nd < 1 || nd > kMaxSpatial)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolutions with %d spatial dimensions are not supported (1..3).", nd);
  if (outer <= 0 || C <= 0 || O <= 0 || group <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid convolution sizes.");
  if (C % group != 0)
    return fail(NBLA_HIP_ERR_VALUE, "Number of input channel needs to be divisible by group. Input channel: %lld, group: %lld.",
                (long long)C, (long long)group);
  if (O % group != 0)
    return fail(NBLA_HIP_ERR_VALUE, "Number of output channel needs to be divisible by group. Output channel: %lld, group: %lld.",
                (long long)O, (long long)group);
  g.outer = outer;
  g.C = C;
  g.O = O;
  g.group = group;
  g.in_sp_size = g.out_sp_size = g.k_size = 1;
  const int shift = kMaxSpatial - nd;
  for (int i = 0; i < kMaxSpatial; ++i) {
    g.in_sp[i] = g.k[i] = g.stride[i] = g.dil[i] = g.out_sp[i] = 1;
    g.pad[i] = 0;
  }
  for (int i = 0; i < nd; ++i) {
    if (kernel[i] <= 0 || stride[i] <= 0 || dil[i] <= 0 || pad[i] < 0 || in_sp[i] <= 0)
      return fail(NBLA_HIP_ERR_VALUE, "invalid convolution parameter at spatial dimension %d.", i);
    const int64_t ke = dil[i] * (kernel[i] - 1) + 1;
    const int64_t span = in_sp[i] + 2 * pad[i] - ke;
    const int64_t o = span / stride[i] + 1;
    if (span < 0 || o <= 0)
      return fail(NBLA_HIP_ERR_VALUE,
                  "Invalid configuration of convolution at %d-th spatial dimension.  {input:%lld, kernel:%lld, "
                  "pad:%lld, stride:%lld, dilation:%lld}.",
                  i, (long long)in_sp[i], (long long)kernel[i], (long long)pad[i], (long long)stride[i],
                  (long long)dil[i]);
    g.in_sp[shift + i] = (int)in_sp[i];
    g.k[shift + i] = (int)kernel[i];
    g.pad[shift + i] = (int)pad[i];
    g.stride[shift + i] = (int)stride[i];
    g.dil[shift + i] = (int)dil[i];
    g.out_sp[shift + i] = (int)o;
    g.in_sp_size *= in_sp[i];
    g.out_sp_size *= o;
    g.k_size *= kernel[i];
  }
  g.Cg = C / group;
  g.Og = O / group;
  g.Kg = g.Cg * g.k_size;
  g.M = outer * g.out_sp_size;
  return NBLA_HIP_OK;
}

namespace {

typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

// ---- digit operand of the unfolded matrix (the int8 bit-weight product)
__device__ __forceinline__ int to_fixed(float v, int s) { return (int)rintf(ldexpf(v, s)); }

// Largest |x| over a slice of the channels of group `grp`, per (sample, input position), as a bit pattern (NaN/Inf
// show as patterns >= 0x7f800000): cmax[slice][position].  Consecutive threads are consecutive positions (coalesced
// for every channel); blockIdx.y is the channel slice.
constexpr int kChannelSlices = 16;
__global__ __launch_bounds__(256) void conv_channel_max(const float *__restrict__ x, uint32_t *__restrict__ cmax,
                                                        ConvGeom g, int64_t grp) {
  const int64_t total = g.outer * g.in_sp_size;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total)
    return;
  const int64_t per = ceil_div(g.Cg, kChannelSlices);
  const int64_t c_begin = blockIdx.y * per, c_end = (c_begin + per < g.Cg) ? c_begin + per : g.Cg;
  const int64_t n = i / g.in_sp_size, p = i - n * g.in_sp_size;
  const float *src = x + (n * g.C + grp * g.Cg) * g.in_sp_size + p;
  uint32_t m = 0u;
  for (int64_t c = c_begin; c < c_end; ++c)
    m = max(m, __float_as_uint(src[c * g.in_sp_size]) & 0x7fffffffu);
  cmax[blockIdx.y * total + i] = m;
}

// One thread per (padded) row of the unfolded matrix: the largest magnitude of the row is the largest channel
// maximum under the kernel window; sets the row's shift and clears its sums.
__global__ __launch_bounds__(256) void conv_row_shift(const uint32_t *__restrict__ cmax, long long *__restrict__ sums,
                                                      int32_t *__restrict__ shift, ConvGeom g, int64_t rows,
                                                      int64_t chunks) {
  const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (m >= rows)
    return;
  for (int64_t c = 0; c < chunks; ++c)
    sums[c * rows + m] = 0;
  if (m >= g.M) {
    shift[m] = 0;
    return;
  }
  const int64_t n = m / g.out_sp_size;
  int64_t p = m - n * g.out_sp_size;
  const int o2 = (int)(p % g.out_sp[2]);
  p /= g.out_sp[2];
  const int o1 = (int)(p % g.out_sp[1]);
  const int o0 = (int)(p / g.out_sp[1]);
  uint32_t amax = 0u;
  for (int k0 = 0; k0 < g.k[0]; ++k0) {
    const int i0 = o0 * g.stride[0] + k0 * g.dil[0] - g.pad[0];
    if ((unsigned)i0 >= (unsigned)g.in_sp[0])
      continue;
    for (int k1 = 0; k1 < g.k[1]; ++k1) {
      const int i1 = o1 * g.stride[1] + k1 * g.dil[1] - g.pad[1];
      if ((unsigned)i1 >= (unsigned)g.in_sp[1])
        continue;
      for (int k2 = 0; k2 < g.k[2]; ++k2) {
        const int i2 = o2 * g.stride[2] + k2 * g.dil[2] - g.pad[2];
        if ((unsigned)i2 >= (unsigned)g.in_sp[2])
          continue;
        const int64_t pos = n * g.in_sp_size + ((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2] + i2;
#pragma unroll
        for (int sl = 0; sl < kChannelSlices; ++sl)
          amax = max(amax, cmax[sl * g.outer * g.in_sp_size + pos]);
      }
    }
  }
  int s = 0;
  if (amax >= 0x7f800000u) {
    s = kBadRow;
  } else if (amax != 0u) {
    s = 22 - binade_exponent(binade_of(amax));
    if (rintf(ldexpf(__uint_as_float(amax), s)) > (float)kDigitMax)
      --s;
  }
  shift[m] = s;
}

// The two kernels above in one launch, for geometries where the input positions under 32 consecutive windows fit a
// small table: a block owns 32 rows of the unfolded matrix (consecutive output positions, so their windows overlap).
// It takes, for every input position the windows can touch -- per run of rows that lie in one sample ("segment") one
// range [lo, hi] of the flattened plane, consecutive lanes on consecutive positions -- the maximum over the channels,
// and a row's largest magnitude is the maximum over its taps' positions.  Same shifts as conv_row_shift gives.
constexpr int kShiftBlock = 1024, kShiftWaves = kShiftBlock / 64, kShiftPixCap = 4096;
__global__ __launch_bounds__(kShiftBlock) void conv_row_shift_windows(const float *__restrict__ x,
                                                                      long long *__restrict__ sums,
                                                                      int32_t *__restrict__ shift, ConvGeom g,
                                                                      int64_t grp, int64_t rows, int64_t chunks) {
  typedef int i32x4_t __attribute__((ext_vector_type(4)));
  __shared__ uint32_t s_pix[kShiftPixCap];
  __shared__ i32x4_t s_taps[64]; // {offset inside the plane, displacements along axes 0 and 1 (16 bits each), axis 2}
  __shared__ int seg_lo[32], seg_hi[32], seg_n[32], row_seg[32], seg_count;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size, taps = (int)g.k_size;
  if (tid < taps) {
    int q = tid;
    const int k2 = q % g.k[2];
    q /= g.k[2];
    const int k1 = q % g.k[1], k0 = q / g.k[1];
    const int e0 = k0 * g.dil[0], e1 = k1 * g.dil[1], e2 = k2 * g.dil[2];
    s_taps[tid] = i32x4_t{(e0 * in1 + e1) * in2 + e2, e0 | (e1 << 16), e2, 0};
  }
  if (tid < 32) {
    seg_lo[tid] = 0x7fffffff;
    seg_hi[tid] = -1;
  }
  for (int i = tid; i < kShiftPixCap; i += kShiftBlock)
    s_pix[i] = 0u;
  // this thread's row (rows past the last one, of the padded operand, get shift 0)
  const int r = lane & 31;
  const int64_t m = (int64_t)blockIdx.x * 32 + r;
  const bool in_range = m < g.M;
  const int64_t n = in_range ? m / g.out_sp_size : 0;
  int p = in_range ? (int)(m - n * g.out_sp_size) : 0;
  const int o2 = p % g.out_sp[2];
  p /= g.out_sp[2];
  const int o1 = p % g.out_sp[1];
  const int o0 = p / g.out_sp[1];
  const int b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
  const int origin = (b0 * in1 + b1) * in2 + b2;
  __syncthreads();
  if (tid < 32) {
    const unsigned long long starts = __ballot(in_range && (r == 0 || m / g.out_sp_size != (m - 1) / g.out_sp_size));
    const int seg = __popcll(starts & ((2ull << r) - 1ull)) - 1;
    row_seg[r] = in_range ? seg : 0;
    if (in_range) {
      int last = 0; // the largest tap offset
      for (int t = 0; t < taps; ++t)
        last = max(last, s_taps[t].x);
      atomicMin(&seg_lo[seg], origin > 0 ? origin : 0);
      atomicMax(&seg_hi[seg], origin + last < plane - 1 ? origin + last : plane - 1);
      seg_n[seg] = (int)n;
    }
    if (r == 0)
      seg_count = __popcll(starts & 0xffffffffull);
  }
  __syncthreads();
  const int nseg = seg_count;
  int my_base = 0, total = 0;
  for (int sgm = 0; sgm < nseg; ++sgm) {
    const int len = seg_hi[sgm] - seg_lo[sgm] + 1;
    if (sgm == row_seg[r])
      my_base = total;
    total += len > 0 ? len : 0;
  }
  // (the host launches this kernel only when every block's positions fit: see conv_row_shift_windows_fits)
  const int Cg = (int)g.Cg;
  int base = 0;
  for (int sgm = 0; sgm < nseg; ++sgm) {
    const int lo = seg_lo[sgm], len = seg_hi[sgm] - lo + 1;
    if (len <= 0)
      continue;
    const float *xs = x + ((int64_t)seg_n[sgm] * g.C + grp * g.Cg) * g.in_sp_size + lo;
    for (int p0 = 0; p0 < len; p0 += 64) {
      const int pix = p0 + lane;
      const bool live = pix < len && base + pix < kShiftPixCap;
      const float *src = xs + (live ? pix : 0);
      uint32_t amax = 0u;
      // channels wave, wave + kShiftWaves, ...: sixteen loads in flight
      for (int c0 = wave; c0 < Cg; c0 += kShiftWaves * 16) {
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int c = c0 + kShiftWaves * j;
          v[j] = src[(int64_t)(c < Cg ? c : wave) * plane];
        }
#pragma unroll
        for (int j = 0; j < 16; ++j)
          if (c0 + kShiftWaves * j < Cg)
            amax = max(amax, __float_as_uint(v[j]) & 0x7fffffffu);
      }
      if (live && amax)
        atomicMax(&s_pix[base + pix], amax);
    }
    base += len;
  }
  __syncthreads();
  if (tid < 32) {
    if (m < rows) {
      for (int64_t c = 0; c < chunks; ++c)
        sums[c * rows + m] = 0;
      uint32_t amax = 0u;
      const int rel = my_base + origin - seg_lo[row_seg[r]];
      for (int t = 0; t < taps; ++t) {
        const i32x4_t e = s_taps[t];
        const int i0 = b0 + (e.y & 0xffff), i1 = b1 + (int)((uint32_t)e.y >> 16), i2 = b2 + e.z;
        if (in_range && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 && (unsigned)i2 < (unsigned)in2)
          amax = max(amax, s_pix[rel + e.x]);
      }
      int sft = 0;
      if (amax >= 0x7f800000u) {
        sft = kBadRow;
      } else if (amax != 0u) {
        sft = 22 - binade_exponent(binade_of(amax));
        if (rintf(ldexpf(__uint_as_float(amax), sft)) > (float)kDigitMax)
          --sft;
      }
      shift[m] = sft;
    }
  }
}

// Whether 32 consecutive windows always touch few enough input positions for conv_row_shift_windows: the positions of
// a run of r windows inside one sample span at most the flattened offset of r - 1 steps of the output walk (whole
// rows / planes of the output counted where the run can cross them) plus the last tap's offset.
bool conv_row_shift_windows_fits(const ConvGeom &g) {
  if (g.k_size > 64 || g.Cg * g.in_sp_size >= ((int64_t)1 << 31))
    return false;
  for (int i = 0; i < kMaxSpatial; ++i)
    if ((int64_t)(g.k[i] - 1) * g.dil[i] >= 65536)
      return false;
  const int64_t r = 32;
  const int64_t d2 = r - 1 < g.out_sp[2] - 1 ? r - 1 : g.out_sp[2] - 1;
  const int64_t c1 = ceil_div(r, (int64_t)g.out_sp[2]), d1 = c1 < g.out_sp[1] - 1 ? c1 : g.out_sp[1] - 1;
  const int64_t c0 = ceil_div(r, (int64_t)g.out_sp[1] * g.out_sp[2]), d0 = c0 < g.out_sp[0] - 1 ? c0 : g.out_sp[0] - 1;
  const int64_t walk = (d0 * g.stride[0] * g.in_sp[1] + d1 * g.stride[1]) * g.in_sp[2] + d2 * g.stride[2];
  const int64_t last = ((int64_t)(g.k[0] - 1) * g.dil[0] * g.in_sp[1] + (int64_t)(g.k[1] - 1) * g.dil[1]) * g.in_sp[2] +
                       (int64_t)(g.k[2] - 1) * g.dil[2];
  int64_t len = walk + last + 1;
  if (len > g.in_sp_size)
    len = g.in_sp_size;
  // a block's rows lie in at most this many samples; every segment may be as long as the bound
  const int64_t segments = ceil_div(r - 1, g.out_sp_size) + 1;
  return len * segments <= kShiftPixCap;
}

// A wavefront converts kTilesPerWave consecutive k tiles of one row block: lane l owns row rb*32 + l%32 and the
// k-slots (l/32)*16 + 0..15 of each tile.  The wavefront first decodes its 64 column indices k -> (channel, tap),
// one per lane, into a wavefront-private LDS table {offset of the tap relative to the window origin, tap
// displacements per dimension, k < Kg}; an element then costs one broadcast table read, three bound checks and one
// load, issued unconditionally from a clamped address and masked afterwards.  Offsets inside one sample's channel
// group are 32-bit (the host checks that they fit).  The row's partial sum of fixed-point values goes to the row sums
// with one 64-bit atomic per lane.
constexpr int kTilesPerWave = 2;
static_assert(kTilesPerWave * kTileK == 64, "one table entry per lane");
__global__ __launch_bounds__(256) void im2col_digits(const float *__restrict__ x, const int32_t *__restrict__ shift,
                                                     long long *__restrict__ sums, uint4_t *__restrict__ out,
                                                     ConvGeom g, int64_t grp, int64_t k_tiles, int64_t tile_groups,
                                                     int64_t rows, int64_t jobs) {
  typedef int i32x4_t __attribute__((ext_vector_type(4)));
  __shared__ i32x4_t table[4][64];
  const int64_t job = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (job >= jobs)
    return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t rb = job / tile_groups, tg = job - rb * tile_groups;
  const int64_t m = rb * kFragRows + (lane & 31);
  const int s = shift[m];
  const bool row_ok = m < g.M && s != kBadRow;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size;
  const int64_t kt_begin = tg * kTilesPerWave;
  {
    const int K0 = g.k[0], K1 = g.k[1], K2 = g.k[2];
    const int kk = (int)(kt_begin * kTileK) + lane;
    int q = kk;
    const int k2 = q % K2;
    q /= K2;
    const int k1 = q % K1;
    q /= K1;
    const int k0 = q % K0, c = q / K0;
    const int e0 = k0 * g.dil[0], e1 = k1 * g.dil[1], e2 = k2 * g.dil[2];
    i32x4_t e;
    e.x = c * plane + (e0 * in1 + e1) * in2 + e2;
    e.y = e0 | (e1 << 16);
    e.z = e2;
    e.w = kk < (int)g.Kg ? 1 : 0;
    table[wave][lane] = e; // read back by this wavefront only: LDS operations of one wavefront complete in order
  }
  // output position of the row (rows past the end read sample 0 and are masked)
  const int64_t n = m < g.M ? m / g.out_sp_size : 0;
  int p = m < g.M ? (int)(m - n * g.out_sp_size) : 0;
  const int o2 = p % g.out_sp[2];
  p /= g.out_sp[2];
  const int o1 = p % g.out_sp[1];
  const int o0 = p / g.out_sp[1];
  const int b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
  const int origin = (b0 * in1 + b1) * in2 + b2; // may be negative; origin + table offset is checked per element
  const float *xn = x + (n * g.C + grp * g.Cg) * g.in_sp_size;
  long long row_sum[2] = {0, 0}; // at most two chunks meet a group of tiles
  for (int t = 0; t < kTilesPerWave; ++t) {
    const int64_t kt = kt_begin + t;
    if (kt >= k_tiles)
      break;
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const i32x4_t e = table[wave][t * kTileK + (lane >> 5) * 16 + j];
      const int i0 = b0 + (e.y & 0xffff), i1 = b1 + (int)((uint32_t)e.y >> 16), i2 = b2 + e.z;
      const bool ok = row_ok && e.w != 0 && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                      (unsigned)i2 < (unsigned)in2;
      const float xv = xn[ok ? origin + e.x : 0];
      v[j] = ok ? xv : 0.0f;
    }
    uint32_t w[3][4];
    int qv[16], part = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      qv[j] = to_fixed(v[j], s); // masked values are 0.0f -> 0 whatever the shift
      part += qv[j];
    }
    pack_digits(qv, w);
    row_sum[(kt * kTileK) / kChunkK - (kt_begin * kTileK) / kChunkK] += part;
    uint4_t *dst = out + ((rb * k_tiles + kt) * kDigits) * 64 + lane;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      uint4_t o;
      o.x = w[d][0], o.y = w[d][1], o.z = w[d][2], o.w = w[d][3];
      dst[d * 64] = o;
    }
  }
  const int64_t chunk0 = (kt_begin * kTileK) / kChunkK;
#pragma unroll
  for (int h = 0; h < 2; ++h)
    if (row_sum[h] != 0)
      atomicAdd(reinterpret_cast<unsigned long long *>(sums + (chunk0 + h) * rows + m), (unsigned long long)row_sum[h]);
}

// ---- the unfolded matrix as the *transposed* digit operand (rows = unfolded columns kk = (channel, tap), contraction
// over the output positions m of all samples): the second factor of the weight gradient dyt^T . col(x).
//
// One shift per channel: the largest |x| of the channel over all samples and positions bounds every unfolded column
// of that channel (a scale only has to bound its row).  Block per channel.
__global__ __launch_bounds__(256) void conv_channel_shift(const float *__restrict__ x, int32_t *__restrict__ shift,
                                                          ConvGeom g, int64_t grp, int64_t rows) {
  __shared__ uint32_t s_max[4];
  const int64_t c = blockIdx.x;
  const int taps = (int)g.k_size;
  uint32_t amax = 0u;
  const float *src = x + (grp * g.Cg + c) * g.in_sp_size;
  const int64_t total = g.outer * g.in_sp_size, sample_stride = g.C * g.in_sp_size;
#pragma unroll 4
  for (int64_t i = threadIdx.x; i < total; i += 256) { // (sample, position) pairs, independent loads
    const int64_t n = i / g.in_sp_size;
    amax = max(amax, __float_as_uint(src[n * sample_stride + (i - n * g.in_sp_size)]) & 0x7fffffffu);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    amax = max(amax, (uint32_t)__shfl_xor((int)amax, off));
  if ((threadIdx.x & 63) == 0)
    s_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3]));
  int s = 0;
  if (amax >= 0x7f800000u) {
    s = kBadRow;
  } else if (amax != 0u) {
    s = 22 - binade_exponent(binade_of(amax));
    if (rintf(ldexpf(__uint_as_float(amax), s)) > (float)kDigitMax)
      --s;
  }
  for (int t = threadIdx.x; t < taps; t += 256)
    shift[c * taps + t] = s;
  if (c == 0) { // padding rows of the operand and its flag word (1: all three digits are in use)
    for (int64_t r = g.Kg + threadIdx.x; r < rows; r += 256)
      shift[r] = 0;
    if (threadIdx.x == 0)
      shift[rows] = 1;
  }
}

// A wavefront converts two k tiles (64 output positions m) of one row block (32 unfolded columns): lane l owns column
// rb*32 + l%32 and the positions (l/32)*16 + 0..15 of each tile.  The 64 positions are decoded once, one per lane,
// into a wavefront-private LDS table {sample base offset (64-bit), window origin per dimension}; the lane's own
// column is decoded once into its tap displacements and channel offset.
__global__ __launch_bounds__(256) void im2col_digits_columns(const float *__restrict__ x,
                                                             const int32_t *__restrict__ shift,
                                                             uint4_t *__restrict__ out, ConvGeom g, int64_t grp,
                                                             int64_t k_tiles, int64_t tile_groups, int64_t jobs) {
  typedef int i32x4_t __attribute__((ext_vector_type(4)));
  __shared__ i32x4_t table[4][64];
  __shared__ int table_b2[4][64];
  const int64_t job = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (job >= jobs)
    return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t rb = job / tile_groups, tg = job - rb * tile_groups;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size;
  const int64_t kt_begin = tg * kTilesPerWave;
  { // this lane's table entry: output position m = kt_begin * 32 + lane
    const int64_t m = kt_begin * kTileK + lane;
    const bool in = m < g.M;
    const int64_t n = in ? m / g.out_sp_size : 0;
    int p = in ? (int)(m - n * g.out_sp_size) : 0;
    const int o2 = p % g.out_sp[2];
    p /= g.out_sp[2];
    const int o1 = p % g.out_sp[1];
    const int o0 = p / g.out_sp[1];
    const int b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
    const int64_t base = (n * g.C + grp * g.Cg) * g.in_sp_size + ((int64_t)b0 * in1 + b1) * in2 + b2;
    i32x4_t e;
    e.x = (int)(uint32_t)(uint64_t)base;
    e.y = (int)(uint32_t)((uint64_t)base >> 32);
    e.z = in ? b0 : -(1 << 30); // a position past the end fails every bound check
    e.w = b1;
    table[wave][lane] = e;
    table_b2[wave][lane] = b2; // read back by this wavefront only: LDS operations of one wavefront complete in order
  }
  // this lane's column kk -> (channel, tap)
  const int64_t kk = rb * kFragRows + (lane & 31);
  const int s = shift[kk];
  const bool row_ok = kk < g.Kg && s != kBadRow;
  int q = row_ok ? (int)kk : 0;
  const int t2 = q % g.k[2];
  q /= g.k[2];
  const int t1 = q % g.k[1];
  q /= g.k[1];
  const int t0 = q % g.k[0], c = q / g.k[0];
  const int e0 = t0 * g.dil[0], e1 = t1 * g.dil[1], e2 = t2 * g.dil[2];
  const int delta = c * plane + (e0 * in1 + e1) * in2 + e2; // offset of the tap relative to the window origin
  for (int t = 0; t < kTilesPerWave; ++t) {
    const int64_t kt = kt_begin + t;
    if (kt >= k_tiles)
      break;
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int idx = t * kTileK + (lane >> 5) * 16 + j;
      const i32x4_t e = table[wave][idx];
      const int b2 = table_b2[wave][idx];
      const int i0 = e.z + e0, i1 = e.w + e1, i2 = b2 + e2;
      const bool ok = row_ok && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                      (unsigned)i2 < (unsigned)in2;
      const int64_t base = (int64_t)(((uint64_t)(uint32_t)e.y << 32) | (uint32_t)e.x);
      const float xv = x[ok ? base + delta : 0];
      v[j] = ok ? xv : 0.0f;
    }
    uint32_t w[3][4];
    int qv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j)
      qv[j] = to_fixed(v[j], s);
    pack_digits(qv, w);
    uint4_t *dst = out + ((rb * k_tiles + kt) * kDigits) * 64 + lane;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      uint4_t o;
      o.x = w[d][0], o.y = w[d][1], o.z = w[d][2], o.w = w[d][3];
      dst[d * 64] = o;
    }
  }
}

// fp32 unfolded matrix [M, Kg] for the general (non bit-representable) path.
__global__ __launch_bounds__(256) void im2col_f32(const float *__restrict__ x, float *__restrict__ col, ConvGeom g,
                                                  int64_t grp, const int *__restrict__ run_if) {
  if (run_if && *run_if == 0) // uniform over the grid
    return;
  const int64_t total = g.M * g.Kg;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / g.Kg;
    col[i] = col_value(x, g, grp, m, i - m * g.Kg);
  }
}

// The same conversion with the gather reduced to one bounds-checked buffer load per element, for kernels of at most
// 64 taps and inputs below 2 GiB.  A block owns one row block and eight consecutive k tiles (two per wavefront).  It
// writes, per row and tap, the byte offset in x of that tap's element of channel 0 -- or an offset past the end of x
// when the tap falls outside the input, the row holds a non-finite value or lies past the last row -- and, per
// column, the byte offset of its channel's plane and its tap (columns past Kg: the tap entry that is never valid).
// An element is then a load at the sum of the two; out-of-range loads return zero, so there are no validity tests
// or selects per element.
constexpr int kRowTaps = 65;
constexpr uint32_t kNowhere = 0x80000000u; // a byte offset past every input this kernel accepts
__global__ __launch_bounds__(256) void im2col_digits_taps(const float *__restrict__ x, const int32_t *__restrict__ shift,
                                                          long long *__restrict__ sums, uint4_t *__restrict__ out,
                                                          ConvGeom g, int64_t grp, int64_t k_tiles,
                                                          int64_t groups_per_row, int64_t rows) {
  typedef int i32x4_t __attribute__((ext_vector_type(4)));
  typedef int i32x2_t __attribute__((ext_vector_type(2)));
  __shared__ i32x4_t s_taps[64];
  __shared__ uint32_t row_taps[32 * kRowTaps];
  __shared__ i32x2_t cols[4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t rb = blockIdx.x / groups_per_row, bg = blockIdx.x - rb * groups_per_row;
  const int64_t kt_begin = (bg * 4 + wave) * kTilesPerWave;
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size, taps = (int)g.k_size;
  if (tid < taps) {
    int q = tid;
    const int k2 = q % g.k[2];
    q /= g.k[2];
    const int k1 = q % g.k[1], k0 = q / g.k[1];
    const int e0 = k0 * g.dil[0], e1 = k1 * g.dil[1], e2 = k2 * g.dil[2];
    s_taps[tid] = i32x4_t{(e0 * in1 + e1) * in2 + e2, e0 | (e1 << 16), e2, 0};
  }
  {
    const int kk = (int)(kt_begin * kTileK) + lane;
    const int c = kk / taps, tap = kk - c * taps;
    const bool live = kk < (int)g.Kg;
    cols[wave][lane] = i32x2_t{live ? c * plane * 4 : 0, live ? tap * 4 : (kRowTaps - 1) * 4};
  }
  // row r = tid % 32 of the block for every thread (the rows' tap offsets are written by eight threads per row)
  const int r = tid & 31;
  const int64_t m = rb * kFragRows + r;
  const int s = shift[m];
  const bool row_ok = m < g.M && s != kBadRow;
  const int64_t n = m < g.M ? m / g.out_sp_size : 0;
  int p = m < g.M ? (int)(m - n * g.out_sp_size) : 0;
  const int o2 = p % g.out_sp[2];
  p /= g.out_sp[2];
  const int o1 = p % g.out_sp[1];
  const int o0 = p / g.out_sp[1];
  const int b0 = o0 * g.stride[0] - g.pad[0], b1 = o1 * g.stride[1] - g.pad[1], b2 = o2 * g.stride[2] - g.pad[2];
  const int origin = (b0 * in1 + b1) * in2 + b2; // may be negative: only taps inside the input are given an offset
  const uint32_t first = (uint32_t)(((n * g.C + grp * g.Cg) * g.in_sp_size + origin) * 4);
  __syncthreads();
  for (int t = tid >> 5; t < taps; t += 8) {
    const i32x4_t e = s_taps[t];
    const int i0 = b0 + (e.y & 0xffff), i1 = b1 + (int)((uint32_t)e.y >> 16), i2 = b2 + e.z;
    const bool ok = row_ok && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 &&
                    (unsigned)i2 < (unsigned)in2;
    row_taps[r * kRowTaps + t] = ok ? first + (uint32_t)e.x * 4u : kNowhere;
  }
  if (tid < 32)
    row_taps[r * kRowTaps + kRowTaps - 1] = kNowhere;
  __syncthreads();
  const uint64_t xbase = reinterpret_cast<uint64_t>(x);
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<void *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(xbase >> 32)) << 32) |
                               (uint32_t)__builtin_amdgcn_readfirstlane((int)xbase)),
      0, __builtin_amdgcn_readfirstlane((int)(g.outer * g.C * g.in_sp_size * 4)), 0x00020000);
  // from here on the lane's row is lane % 32 (the same as tid % 32) and its k-slots (lane / 32) * 16 + 0..15
  const uint32_t *my_taps = row_taps + r * kRowTaps;
  long long row_sum[2] = {0, 0}; // at most two chunks meet a group of tiles
  for (int t = 0; t < kTilesPerWave; ++t) {
    const int64_t kt = kt_begin + t;
    if (kt >= k_tiles)
      break;
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const i32x2_t e = cols[wave][t * kTileK + (lane >> 5) * 16 + j];
      const uint32_t at = my_taps[e.y >> 2] + (uint32_t)e.x;
      v[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(xrsrc, (int)at, 0, 0));
    }
    uint32_t w[3][4];
    int qv[16], part = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      qv[j] = to_fixed(v[j], row_ok ? s : 0); // elements that are not read are 0.0f -> 0 whatever the shift
      part += qv[j];
    }
    pack_digits(qv, w);
    row_sum[(kt * kTileK) / kChunkK - (kt_begin * kTileK) / kChunkK] += part;
    uint4_t *dst = out + ((rb * k_tiles + kt) * kDigits) * 64 + lane;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      uint4_t o;
      o.x = w[d][0], o.y = w[d][1], o.z = w[d][2], o.w = w[d][3];
      dst[d * 64] = o;
    }
  }
  const int64_t chunk0 = (kt_begin * kTileK) / kChunkK;
#pragma unroll
  for (int h = 0; h < 2; ++h)
    if (row_sum[h] != 0)
      atomicAdd(reinterpret_cast<unsigned long long *>(sums + (chunk0 + h) * rows + m), (unsigned long long)row_sum[h]);
}

} // namespace

// `scratch` holds kChannelSlices * outer * in_sp_size uint32 (the channel maxima).
int launch_im2col_digits(const float *x, void *xdigits, void *scratch, const ConvGeom &g, int64_t grp,
                         hipStream_t stream) {
  // the unfold kernel keeps offsets inside one sample's channel group, output positions and k in 32 bits
  bool fits = g.Cg * g.in_sp_size < ((int64_t)1 << 31) && g.out_sp_size < ((int64_t)1 << 31) &&
              g.Kg + 2 * kTileK * kTilesPerWave < ((int64_t)1 << 31);
  for (int i = 0; i < kMaxSpatial; ++i)
    fits = fits && (int64_t)(g.k[i] - 1) * g.dil[i] < 65536; // tap displacements travel as 16-bit fields
  if (!fits)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution: a sample's channel group, its output map or the unfolded "
                                              "row has 2^31 elements or more, or a dilated kernel spans 65536.");
  const DigitOperand d = digit_operand(g.M, g.Kg);
  char *base = static_cast<char *>(xdigits);
  long long *sums = reinterpret_cast<long long *>(base + d.sum_off);
  int32_t *shift = reinterpret_cast<int32_t *>(base + d.shift_off);
  if (conv_row_shift_windows_fits(g)) {
    hipLaunchKernelGGL(conv_row_shift_windows, dim3((unsigned)d.row_blocks), dim3(kShiftBlock), 0, stream, x, sums,
                       shift, g, grp, d.rows, d.chunks);
    NBLA_HIP_LAUNCH_CHECK("conv_row_shift_windows");
  } else {
    uint32_t *cmax = static_cast<uint32_t *>(scratch);
    hipLaunchKernelGGL(conv_channel_max, dim3((unsigned)ceil_div(g.outer * g.in_sp_size, 256), kChannelSlices),
                       dim3(256), 0, stream, x, cmax, g, grp);
    NBLA_HIP_LAUNCH_CHECK("conv_channel_max");
    hipLaunchKernelGGL(conv_row_shift, dim3((unsigned)ceil_div(d.rows, 256)), dim3(256), 0, stream, cmax, sums, shift,
                       g, d.rows, d.chunks);
    NBLA_HIP_LAUNCH_CHECK("conv_row_shift");
  }
  if (g.k_size <= 64 && g.outer * g.C * g.in_sp_size * 4 < ((int64_t)1 << 31)) {
    const int64_t groups_per_row = ceil_div(d.k_tiles, 4 * kTilesPerWave);
    hipLaunchKernelGGL(im2col_digits_taps, dim3((unsigned)(d.row_blocks * groups_per_row)), dim3(256), 0, stream, x,
                       shift, sums, reinterpret_cast<uint4_t *>(base), g, grp, d.k_tiles, groups_per_row, d.rows);
    NBLA_HIP_LAUNCH_CHECK("im2col_digits_taps");
    return NBLA_HIP_OK;
  }
  const int64_t tile_groups = ceil_div(d.k_tiles, kTilesPerWave), jobs = d.row_blocks * tile_groups;
  hipLaunchKernelGGL(im2col_digits, dim3((unsigned)ceil_div(jobs, 4)), dim3(256), 0, stream, x, shift, sums,
                     reinterpret_cast<uint4_t *>(base), g, grp, d.k_tiles, tile_groups, d.rows, jobs);
  NBLA_HIP_LAUNCH_CHECK("im2col_digits");
  return NBLA_HIP_OK;
}

// Digit operand of col(x)^T: rows = the Kg unfolded columns, contraction over the M output positions.
int launch_im2col_digits_columns(const float *x, void *digits, const ConvGeom &g, int64_t grp, hipStream_t stream) {
  bool fits = g.Cg * g.in_sp_size < ((int64_t)1 << 31) && g.out_sp_size < ((int64_t)1 << 31) &&
              g.Kg < ((int64_t)1 << 31);
  for (int i = 0; i < kMaxSpatial; ++i)
    fits = fits && (int64_t)g.in_sp[i] + g.pad[i] + (int64_t)g.k[i] * g.dil[i] < ((int64_t)1 << 30);
  if (!fits)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution backward: a sample's channel group, its output map or a "
                                              "padded input extent has 2^30 elements or more.");
  const DigitOperand d = digit_operand(g.Kg, g.M);
  char *base = static_cast<char *>(digits);
  int32_t *shift = reinterpret_cast<int32_t *>(base + d.shift_off);
  hipLaunchKernelGGL(conv_channel_shift, dim3((unsigned)g.Cg), dim3(256), 0, stream, x, shift, g, grp, d.rows);
  NBLA_HIP_LAUNCH_CHECK("conv_channel_shift");
  const int64_t tile_groups = ceil_div(d.k_tiles, kTilesPerWave), jobs = d.row_blocks * tile_groups;
  hipLaunchKernelGGL(im2col_digits_columns, dim3((unsigned)ceil_div(jobs, 4)), dim3(256), 0, stream, x, shift,
                     reinterpret_cast<uint4_t *>(base), g, grp, d.k_tiles, tile_groups, jobs);
  NBLA_HIP_LAUNCH_CHECK("im2col_digits_columns");
  return NBLA_HIP_OK;
}

int launch_im2col_f32(const float *x, float *col, const ConvGeom &g, int64_t grp, hipStream_t stream,
                      const int *run_if) {
  int64_t blocks = ceil_div(g.M * g.Kg, 256);
  if (blocks > 65536)
    blocks = 65536;
  hipLaunchKernelGGL(im2col_f32, dim3((unsigned)blocks), dim3(256), 0, stream, x, col, g, grp, run_if);
  NBLA_HIP_LAUNCH_CHECK("im2col_f32");
  return NBLA_HIP_OK;
}

namespace {

// Windows holding a NaN or an infinity (shift[m] == kBadRow): the digit products leave NaN in all their outputs, while
// the reference's product propagates such values output by output (convolution.cpp:185-193: the row of the unfolded
// input times Ws = Wb * alpha, then + b: Inf * w = +-Inf, Inf - Inf = NaN).  Those windows -- rare -- are recomputed
// here as plain fp32 dot products over the materialised signs of the group, Wbg [Og, Kg]; yg is the group's first
// output map.  A block looks at 256 marks at a time and leaves at once when none of them is set.
__global__ __launch_bounds__(256) void conv_redo_marked_windows(const float *__restrict__ x,
                                                                const float *__restrict__ Wbg,
                                                                const float *__restrict__ alpha,
                                                                const float *__restrict__ bias, float *__restrict__ yg,
                                                                const int32_t *__restrict__ shift, ConvGeom g,
                                                                int64_t grp) {
  for (int64_t base = (int64_t)blockIdx.x * 256; base < g.M; base += (int64_t)gridDim.x * 256) {
    const int64_t mine = base + threadIdx.x;
    const int marked = mine < g.M && shift[mine] == kBadRow;
    if (!__syncthreads_or(marked))
      continue;
    const int64_t end = base + 256 < g.M ? base + 256 : g.M;
    for (int64_t m = base; m < end; ++m) {
      if (shift[m] != kBadRow) // uniform over the block
        continue;
      const int64_t n = m / g.out_sp_size, pos = m - n * g.out_sp_size;
      for (int64_t o = threadIdx.x; o < g.Og; o += 256) {
        const float a = alpha ? alpha[o] : 1.0f;
        float acc = 0.0f;
        for (int64_t k = 0; k < g.Kg; ++k) {
          const float w = alpha ? Wbg[o * g.Kg + k] * a : Wbg[o * g.Kg + k]; // the scaled weight of the reference
          acc = acc + col_value(x, g, grp, m, k) * w;
        }
        yg[(n * g.O + o) * g.out_sp_size + pos] = bias ? acc + bias[o] : acc;
      }
    }
  }
}

int launch_conv_redo(const float *x, const float *Wbg, const float *alpha, const float *bias, float *yg,
                     const int32_t *shift, const ConvGeom &g, int64_t grp, hipStream_t stream) {
  int64_t blocks = ceil_div(g.M, 256);
  if (blocks > 1024)
    blocks = 1024;
  hipLaunchKernelGGL(conv_redo_marked_windows, dim3((unsigned)blocks), dim3(256), 0, stream, x, Wbg, alpha, bias, yg,
                     shift, g, grp);
  NBLA_HIP_LAUNCH_CHECK("conv_redo_marked_windows");
  return NBLA_HIP_OK;
}

struct ConvWorkspace {
  size_t bits_off, bits_stride, split_off, cmax_off, prep_off, count_off, tap_bits_off, tap_bits_stride, col_off, total;
};

ConvWorkspace plan_conv(const ConvGeom &g) {
  ConvWorkspace w;
  size_t off = 0;
  w.bits_off = off;
  w.bits_stride = round_up(nbla_hip_packed_bits_bytes(g.Kg, g.Og), 256);
  off += w.bits_stride * g.group;
  w.split_off = off;
  off += round_up(nbla_hip_digit_operand_bytes(g.M, g.Kg), 256);
  w.cmax_off = off;
  off += round_up((size_t)16 * g.outer * g.in_sp_size * sizeof(uint32_t), 256); // kChannelSlices slices
  w.prep_off = off;
  off += round_up(nbla_hip_binarize_workspace_bytes(g.Kg, g.Og), 256);
  w.count_off = off;
  off += round_up(sizeof(int) * g.group, 256);
  w.tap_bits_off = off; // the weights prepared for the product over input positions held in LDS, when that runs
  w.tap_bits_stride = round_up(conv_slab_prepared_bytes(g), 256);
  off += w.tap_bits_stride * g.group;
  w.col_off = off; // fp32 unfolded matrix of the general path shares the split operand's space when it fits
  w.total = off;
  return w;
}

int binary_conv_forward(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                        const ConvGeom &g, float zero_to, void *workspace, size_t workspace_bytes, void *stream_) {
  const ConvWorkspace ws = plan_conv(g);
  const bool representable = (zero_to == 1.0f || zero_to == -1.0f);
  const size_t col_bytes = representable ? 0 : round_up((size_t)g.M * g.Kg * sizeof(float), 256);
  if (workspace_bytes < ws.total + col_bytes || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "binary convolution workspace too small (%zu < %zu) or misaligned.",
                workspace_bytes, ws.total + col_bytes);
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  if (conv_direct_forward_applies(g)) { // many small groups: all of them in one launch each, over the materialised signs
    rc = launch_conv_direct_binarize(W, Wb, alpha, g, zero_to, stream);
    if (rc)
      return rc;
    return launch_conv_direct_forward(x, Wb, alpha, bias, y, g, stream);
  }
  char *base = static_cast<char *>(workspace);
  int *counts = reinterpret_cast<int *>(base + ws.count_off);
  const bool slab = conv_slab_applies(g);
  // weights: per group a [Og, Kg] slab stored n-major -> packed [Kg, Og] bits, Sign, alpha (the product over input
  // positions held in LDS prepares its own form of the weights, below)
  for (int64_t grp = 0; grp < g.group && !slab; ++grp) {
    const int64_t woff = grp * g.Og * g.Kg;
    rc = nbla_hip_binarize_weights_f32(W + woff, Wb + woff, alpha ? alpha + grp * g.Og : nullptr,
                                       reinterpret_cast<uint32_t *>(base + ws.bits_off + grp * ws.bits_stride), g.Kg,
                                       g.Og, 1, zero_to, representable ? nullptr : counts + grp, base + ws.prep_off,
                                       nbla_hip_binarize_workspace_bytes(g.Kg, g.Og), stream_);
    if (rc)
      return rc;
  }
  // Sign(0) = zero_to that is neither +1 nor -1 cannot be a sign bit: the matrix-core product of a group is then only
  // valid when the group holds no weight that is neither negative nor positive.  The binarising pass has counted such
  // weights on the device; the fp32 product over the materialised signs (unfold + product) is launched behind the
  // matrix-core one with that count as its go-ahead and replaces the group's outputs when it is non-zero.  The host
  // never reads the count.
  const int64_t hw = g.out_sp_size;
  for (int64_t grp = 0; grp < g.group; ++grp) {
    float *yg = y + grp * g.Og * hw;
    const float *ag = alpha ? alpha + grp * g.Og : nullptr;
    const float *bg = bias ? bias + grp * g.Og : nullptr;
    if (slab) {
      void *prepared = base + ws.tap_bits_off + grp * ws.tap_bits_stride;
      rc = launch_conv_slab_prepare(W + grp * g.Og * g.Kg, Wb + grp * g.Og * g.Kg, prepared, g, zero_to, stream);
      if (rc)
        return rc;
      rc = launch_conv_slab(x, g, grp, prepared, alpha ? alpha + grp * g.Og : nullptr,
                            representable ? nullptr : counts + grp, bg, y, stream, nullptr, false,
                            Wb + grp * g.Og * g.Kg);
    } else {
      // the rows' marks sit where the digit operand keeps its scale exponents (the fused unfold has no other use for
      // that space)
      int32_t *shift = reinterpret_cast<int32_t *>(base + ws.split_off + digit_operand(g.M, g.Kg).shift_off);
      if (gemm_bits_unfold_applies(g)) {
        rc = launch_gemm_bits_unfold(x, g, grp,
                                     reinterpret_cast<const uint32_t *>(base + ws.bits_off + grp * ws.bits_stride), ag,
                                     bg, yg, stream, shift);
      } else {
        rc = launch_im2col_digits(x, base + ws.split_off, base + ws.cmax_off, g, grp, stream);
        if (rc)
          return rc;
        rc = launch_gemm_bits(base + ws.split_off,
                              reinterpret_cast<const uint32_t *>(base + ws.bits_off + grp * ws.bits_stride), ag, bg,
                              yg, g.M, g.Kg, g.Og, hw, g.O * hw, hw, true, stream);
      }
      if (rc)
        return rc;
      rc = launch_conv_redo(x, Wb + grp * g.Og * g.Kg, ag, bg, yg, shift, g, grp, stream);
    }
    if (rc)
      return rc;
    if (!representable) {
      float *col = reinterpret_cast<float *>(base + ws.total);
      rc = launch_im2col_f32(x, col, g, grp, stream, counts + grp);
      if (rc)
        return rc;
      rc = launch_gemm_f32_mapped(col, Wb + grp * g.Og * g.Kg, true, ag, bg, yg, g.M, g.Kg, g.Og, hw, g.O * hw, hw,
                                  stream, counts + grp);
      if (rc)
        return rc;
    }
  }
  return NBLA_HIP_OK;
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_convolution_output_shape(int nd, const int64_t *in_sp, const int64_t *kernel, const int64_t *pad,
                                      const int64_t *stride, const int64_t *dilation, int64_t *out_sp) {
  ConvGeom g;
  const int rc = make_geom(g, 1, 1, nd, in_sp, 1, kernel, pad, stride, dilation, 1);
  if (rc)
    return rc;
  for (int i = 0; i < nd; ++i)
    out_sp[i] = g.out_sp[kMaxSpatial - nd + i];
  return NBLA_HIP_OK;
}

size_t nbla_hip_binary_convolution_workspace_bytes(int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                                   const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                                   const int64_t *dilation, int64_t group, float quantize_zero_to) {
  ConvGeom g;
  if (make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group))
    return 0;
  const bool representable = (quantize_zero_to == 1.0f || quantize_zero_to == -1.0f);
  return plan_conv(g).total + (representable ? 0 : round_up((size_t)g.M * g.Kg * sizeof(float), 256));
}

int nbla_hip_binary_convolution_slab_plan(int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                          const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                          const int64_t *dilation, int64_t group, int32_t *plan) {
  if (!plan)
    return fail(NBLA_HIP_ERR_VALUE, "slab plan: no output array.");
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  plan[0] = plan[1] = plan[2] = plan[3] = 0;
  conv_slab_plan_summary(g, plan);
  return NBLA_HIP_OK;
}

int nbla_hip_binary_weight_convolution_f32(const float *x, const float *W, float *Wb, float *alpha, const float *bias,
                                           float *y, int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                           const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                           const int64_t *dilation, int64_t group, float quantize_zero_to,
                                           void *workspace, size_t workspace_bytes, void *stream) {
  if (!alpha)
    return fail(NBLA_HIP_ERR_VALUE, "BinaryWeightConvolution needs an alpha output of size channels_o.");
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  return binary_conv_forward(x, W, Wb, alpha, bias, y, g, quantize_zero_to, workspace, workspace_bytes, stream);
}

int nbla_hip_binary_connect_convolution_f32(const float *x, const float *W, float *Wb, const float *bias, float *y,
                                            int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                            const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                            const int64_t *dilation, int64_t group, float quantize_zero_to,
                                            void *workspace, size_t workspace_bytes, void *stream) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  return binary_conv_forward(x, W, Wb, nullptr, bias, y, g, quantize_zero_to, workspace, workspace_bytes, stream);
}

} // extern "C"
