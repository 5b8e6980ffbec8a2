// Convolutions in plain fp32 on the vector units, for the geometries the matrix-core paths serve badly: grouped
// convolutions with small groups (depthwise, ResNeXt-style), where every group's product is far too small for the
// matrix cores and the general path pays several launches per group (256 groups of a depthwise layer: milliseconds
// of launches around microseconds of work), and single groups of few channels (a network's first layers).  All groups
// in one launch per kernel, straight from x, dy and the weights without an unfolded matrix
// (convolution.cpp:161-197 forward, :199-330 backward: per sample and group an unfold and a product):
//   conv_direct_forward_tile   forward (and, on transposed weights, the input gradient of unit stride) with 8 or 16
//                              channels of the result per thread, the weights in LDS
//   conv_direct_gather         forward and input gradient, a thread per element, for everything else
//   conv_direct_dw_pairs / conv_direct_dw_tile   weight gradient: sums per thread, or tiles of 64 x 64 weights
//   conv_direct_db_chunks      bias gradient
// and one-thread-per-element forms (conv_direct_forward, conv_direct_dw, conv_direct_db) for what exceeds those kernels'
// limits.  The same kernels serve the binary convolutions: the weights are then the materialised signs, multiplied by
// alpha[o] as binary_weight_convolution.cpp:100-110 forms Ws.
#include "common.hpp"
#include "conv_geom.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

constexpr int kDirectBlock = 256;

struct Position {
  int o0, o1, o2;
};
__device__ __forceinline__ Position out_position(const ConvGeom &g, int64_t p) {
  Position q;
  q.o2 = (int)(p % g.out_sp[2]);
  p /= g.out_sp[2];
  q.o1 = (int)(p % g.out_sp[1]);
  q.o0 = (int)(p / g.out_sp[1]);
  return q;
}

// y[n, o, p] = sum_k x[n, c(k), window(p, tap(k))] * w[o, k] (* scale[o]) (+ bias[o]); zeros where the window leaves
// the input (they are multiplied like any other value: 0 * Inf = NaN as in the reference's product).
__global__ __launch_bounds__(kDirectBlock) void conv_direct_forward(const float *__restrict__ x,
                                                                    const float *__restrict__ w,
                                                                    const float *__restrict__ scale,
                                                                    const float *__restrict__ bias,
                                                                    float *__restrict__ y, ConvGeom g) {
  const int64_t total = g.outer * g.O * g.out_sp_size;
  for (int64_t i = (int64_t)blockIdx.x * kDirectBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kDirectBlock) {
    const int64_t p = i % g.out_sp_size, no = i / g.out_sp_size;
    const int64_t o = no % g.O, n = no / g.O, grp = o / g.Og;
    const Position q = out_position(g, p);
    const int b0 = q.o0 * g.stride[0] - g.pad[0], b1 = q.o1 * g.stride[1] - g.pad[1], b2 = q.o2 * g.stride[2] - g.pad[2];
    const float *xn = x + (n * g.C + grp * g.Cg) * g.in_sp_size;
    const float *wo = w + o * g.Kg;
    const float a = scale ? scale[o] : 1.0f;
    float acc = 0.0f;
    for (int64_t c = 0; c < g.Cg; ++c) {
      const float *xc = xn + c * g.in_sp_size;
      const float *wc = wo + c * g.k_size;
      int t = 0;
      for (int k0 = 0; k0 < g.k[0]; ++k0)
        for (int k1 = 0; k1 < g.k[1]; ++k1)
          for (int k2 = 0; k2 < g.k[2]; ++k2, ++t) {
            const int i0 = b0 + k0 * g.dil[0], i1 = b1 + k1 * g.dil[1], i2 = b2 + k2 * g.dil[2];
            const bool in = (unsigned)i0 < (unsigned)g.in_sp[0] && (unsigned)i1 < (unsigned)g.in_sp[1] &&
                            (unsigned)i2 < (unsigned)g.in_sp[2];
            const float xv = in ? xc[((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2] + i2] : 0.0f;
            const float wv = scale ? wc[t] * a : wc[t];
            acc = acc + xv * wv;
          }
    }
    y[i] = bias ? acc + bias[o] : acc;
  }
}

// The same for kOut consecutive output channels of one group per thread (Og a multiple of kOut): a block is one
// (sample, tile of channels) and 256 output positions.  The tile's weights (times alpha) are laid out [k][channel] in
// LDS once per block, so a tap's kOut weights are kOut / 4 broadcast reads of 16 bytes, and every input value loaded
// serves kOut products; the loads of four taps along the innermost kernel axis are issued together.
constexpr int kDirectLdsFloats = 12288; // 48 KiB of weights per block
// kDrop: a tap outside the input contributes nothing (it reads a row of zero weights) instead of 0 * weight: the
// form in which the kernel computes an input gradient (see launch_conv_direct_dx), where the reference never
// forms those products.  accum: the result is added to y.
template <int kOut, bool kDrop>
__global__ __launch_bounds__(kDirectBlock) void conv_direct_forward_tile(const float *__restrict__ x,
                                                                         const float *__restrict__ w,
                                                                         const float *__restrict__ scale,
                                                                         const float *__restrict__ bias,
                                                                         float *__restrict__ y, ConvGeom g, int accum) {
  extern __shared__ __attribute__((aligned(16))) float s_w[]; // [Kg (+ 1 row of zeros)][kOut]
  typedef float float4_d __attribute__((ext_vector_type(4)));
  const int64_t otiles = g.O / kOut;
  const int64_t n = blockIdx.y / otiles, o0 = (blockIdx.y - n * otiles) * kOut, grp = o0 / g.Og;
  const int Kg = (int)g.Kg;
  for (int i = threadIdx.x; i < Kg * kOut; i += kDirectBlock) {
    const int j = i / Kg, k = i - j * Kg; // consecutive threads read consecutive k of one channel
    const float wv = w[(o0 + j) * g.Kg + k];
    s_w[k * kOut + j] = scale ? wv * scale[o0 + j] : wv; // Ws = Wb * alpha, rounded once as the reference forms it
  }
  if (kDrop && threadIdx.x < kOut)
    s_w[Kg * kOut + threadIdx.x] = 0.0f;
  __syncthreads();
  const int64_t p = (int64_t)blockIdx.x * kDirectBlock + threadIdx.x;
  const bool live = p < g.out_sp_size;
  const Position q = out_position(g, live ? p : 0);
  const int b0 = q.o0 * g.stride[0] - g.pad[0], b1 = q.o1 * g.stride[1] - g.pad[1], b2 = q.o2 * g.stride[2] - g.pad[2];
  const float *xn = x + (n * g.C + grp * g.Cg) * g.in_sp_size;
  float acc[kOut];
#pragma unroll
  for (int j = 0; j < kOut; ++j)
    acc[j] = 0.0f;
  int t = 0; // k = c * k_size + tap
  for (int64_t c = 0; c < g.Cg; ++c) {
    const float *xc = xn + c * g.in_sp_size;
    for (int k0 = 0; k0 < g.k[0]; ++k0)
      for (int k1 = 0; k1 < g.k[1]; ++k1) {
        const int i0 = b0 + k0 * g.dil[0], i1 = b1 + k1 * g.dil[1];
        const bool row_in = live && (unsigned)i0 < (unsigned)g.in_sp[0] && (unsigned)i1 < (unsigned)g.in_sp[1];
        const float *xr = xc + ((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2];
        for (int k2 = 0; k2 < g.k[2]; k2 += 4) {
          float xv[4];
          bool in[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int i2 = b2 + (k2 + u) * g.dil[2];
            in[u] = row_in && k2 + u < g.k[2] && (unsigned)i2 < (unsigned)g.in_sp[2];
            xv[u] = in[u] ? xr[i2] : 0.0f;
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            if (k2 + u < g.k[2]) { // uniform
              const float4_d *wk =
                  reinterpret_cast<const float4_d *>(s_w + (kDrop && !in[u] ? Kg : t + u) * kOut);
#pragma unroll
              for (int j4 = 0; j4 < kOut / 4; ++j4) {
                const float4_d wv = wk[j4];
                acc[4 * j4 + 0] = acc[4 * j4 + 0] + xv[u] * wv.x;
                acc[4 * j4 + 1] = acc[4 * j4 + 1] + xv[u] * wv.y;
                acc[4 * j4 + 2] = acc[4 * j4 + 2] + xv[u] * wv.z;
                acc[4 * j4 + 3] = acc[4 * j4 + 3] + xv[u] * wv.w;
              }
            }
          }
          t += (g.k[2] - k2 < 4) ? g.k[2] - k2 : 4;
        }
      }
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < kOut; ++j)
    {
      float *out = y + (n * g.O + o0 + j) * g.out_sp_size + p;
      const float v = bias ? acc[j] + bias[o0 + j] : acc[j];
      *out = accum ? *out + v : v;
    }
  }
}

// The weights of the convolution that computes an input gradient of unit stride: channels' roles exchanged within
// each group, taps reversed, signs taken and alpha folded in:
//   wt[grp * Cg + c][o * taps + (taps - 1 - t)] = f(w[grp * Og + o][c * taps + t])
__global__ __launch_bounds__(kDirectBlock) void conv_direct_transpose_weights(const float *__restrict__ w,
                                                                              const float *__restrict__ scale,
                                                                              float *__restrict__ wt, int64_t count,
                                                                              int Og, int Cg, int taps, int take_sign,
                                                                              float zero_to) {
  const int64_t i = (int64_t)blockIdx.x * kDirectBlock + threadIdx.x;
  if (i >= count)
    return;
  const int t = (int)(i % taps);
  const int64_t oc = i / taps, c = oc % Cg, og = oc / Cg, grp = og / Og, o = og - grp * Og; // og: channel out, global
  float wv = w[i];
  if (take_sign)
    wv = (wv > 0.0f) ? 1.0f : ((wv < 0.0f) ? -1.0f : zero_to);
  if (scale)
    wv = wv * scale[og];
  wt[((grp * Cg + c) * Og + o) * taps + (taps - 1 - t)] = wv;
}

// One batch of taps of one element of the result: rows the sample's source at the first of kOB channels (the next ones
// L floats further, as many as `channels`), sw those channels' weights in LDS ([channel][taps], this batch's first tap),
// reach/ok where the taps land (byte offsets into a channel of the source).  The loads of a batch are all in flight together;
// taps outside the output load a valid address and are left out of the sum.  kB: taps per batch (the first kB entries
// of reach / ok); kFull: all kB taps exist.
constexpr int kTapBatch = 9;
constexpr uint32_t kNoReach = 0xffffffffu;
template <int kOB, int kB, bool kFull, bool kForward>
__device__ __forceinline__ float conv_direct_gather_batch(const float *__restrict__ rows, int64_t L, const float *sw, int taps,
                                                      int channels, int count, const uint32_t (&reach)[kTapBatch],
                                                      const bool (&ok)[kTapBatch], float acc) {
  float gy[kOB][kB];
#pragma unroll
  for (int jo = 0; jo < kOB; ++jo) {
    const char *row = reinterpret_cast<const char *>(rows + (jo < channels ? jo : channels - 1) * L);
#pragma unroll
    for (int j = 0; j < kB; ++j)
      gy[jo][j] = *reinterpret_cast<const float *>(row + reach[j]);
  }
#pragma unroll
  for (int jo = 0; jo < kOB; ++jo) {
    const bool live = jo < channels;
    const float *wr = sw + (live ? jo : channels - 1) * taps;
#pragma unroll
    for (int j = 0; j < kB; ++j) {
      const float wv = wr[kFull || j < count ? j : 0];
      if (kForward) // a tap in the padding is a zero that is multiplied
        acc = acc + (live ? (ok[j] ? gy[jo][j] : 0.0f) * wv : 0.0f);
      else
        acc = acc + (live && ok[j] ? gy[jo][j] * wv : 0.0f);
    }
  }
  return acc;
}

// Both directions of a convolution of small groups as a gather, a thread per element of the result:
//   backward  dx[n, c, q] (+)= sum over the group's o and the taps whose window position p lies in the output of
//             (dy[n, o, p] * scale[o]) * w[o, c, tap]   (the unfolded gradient folded back, convolution.cpp:262-283);
//             take_sign: w holds the real-valued weights of a binary convolution, whose signs (sign.hpp:48-50) are
//             what the forward pass multiplied with;
//   forward   y[n, o, p] = sum over the group's c and the taps of x[n, c, window(p, tap)] * (w[o, c, tap] * scale[o])
//             (+ bias[o]); zeros where the window leaves the input, multiplied like any other value (0 * Inf = NaN as
//             in the reference's product).
// Block (tile of the result's positions, channels, samples), of 64 to 256 threads.  Where each tap lands from a
// thread's position is the same for every (sample, channel) the block visits: a table in LDS, filled once (held in
// registers when the kernel has at most kTapBatch taps).  The weights that meet one channel of the result, `held`
// source channels at a time, signs taken and scaled, sit in LDS too; the samples' loop runs inside, so they are
// prepared once per channel.  32-bit arithmetic per lane: a block-uniform row pointer plus a byte offset.
// kUnit (backward): unit strides, no divisibility to test; kClasses (backward, strides): see below.
template <bool kForward, bool kUnit, bool kClasses>
__global__ __launch_bounds__(kDirectBlock) void conv_direct_gather(const float *__restrict__ src,
                                                                   const float *__restrict__ w,
                                                                   const float *__restrict__ scale,
                                                                   const float *__restrict__ bias,
                                                                   float *__restrict__ dst, ConvGeom g, int held,
                                                                   int accum, int take_sign, float zero_to) {
  constexpr int kOB = 1; // (more source channels per step gave nothing)
  extern __shared__ uint32_t s_gather[];
  const int all_taps = (int)g.k_size, threads = (int)blockDim.x, tid = (int)threadIdx.x;
  uint32_t *s_reach = s_gather;                                              // [taps][threads]: byte offset, or kNoReach
  float *s_w = reinterpret_cast<float *>(s_gather + (size_t)all_taps * threads); // [held][taps]
  int *s_tap = reinterpret_cast<int *>(s_w + (size_t)held * all_taps);        // [taps]: which taps the block uses
  const int64_t positions = kForward ? g.out_sp_size : g.in_sp_size, L = kForward ? g.in_sp_size : g.out_sp_size;
  const int in0 = (int)g.in_sp[0], in1 = (int)g.in_sp[1], in2 = (int)g.in_sp[2], out0 = (int)g.out_sp[0],
            out1 = (int)g.out_sp[1], out2 = (int)g.out_sp[2];
  const int s0 = (int)g.stride[0], s1 = (int)g.stride[1], s2 = (int)g.stride[2];
  int pos, q0, q1, q2, r0 = 0, r1 = 0, r2 = 0, taps = all_taps;
  bool live;
  if (!kClasses) {
    pos = (int)(blockIdx.x * blockDim.x) + tid;
    live = pos < positions;
    const int d1 = kForward ? out1 : in1, d2 = kForward ? out2 : in2;
    const int r = pos / d2;
    q2 = pos % d2, q1 = r % d1, q0 = r / d1;
  } else {
    // A strided convolution reaches an input position only through the taps that match the position's remainders
    // modulo the strides.  A block takes positions of one class of remainders (r0, r1, r2), so that all its threads
    // use the same taps, and keeps only those: 1/(s0 s1 s2) of the kernel on average.
    const int tiles = (int)gridDim.x / (s0 * s1 * s2), cls = (int)blockIdx.x / tiles, tile = (int)blockIdx.x - cls * tiles;
    r2 = cls % s2, r1 = (cls / s2) % s1, r0 = cls / (s2 * s1);
    const int u0n = in0 > r0 ? (in0 - r0 + s0 - 1) / s0 : 0, u1n = in1 > r1 ? (in1 - r1 + s1 - 1) / s1 : 0,
              u2n = in2 > r2 ? (in2 - r2 + s2 - 1) / s2 : 0;
    const int li = tile * threads + tid;
    live = li < u0n * u1n * u2n;
    const int v = li / (u2n > 0 ? u2n : 1);
    q2 = r2 + s2 * (li - v * (u2n > 0 ? u2n : 1));
    q1 = r1 + s1 * (v % (u1n > 0 ? u1n : 1)), q0 = r0 + s0 * (v / (u1n > 0 ? u1n : 1));
    pos = (q0 * in1 + q1) * in2 + q2;
  }
  {
    int t = 0, used = 0;
    for (int k0 = 0; k0 < (int)g.k[0]; ++k0)
      for (int k1 = 0; k1 < (int)g.k[1]; ++k1)
        for (int k2 = 0; k2 < (int)g.k[2]; ++k2, ++t) {
          uint32_t at = kNoReach;
          if (kForward) {
            const int i0 = q0 * s0 - (int)g.pad[0] + k0 * (int)g.dil[0], i1 = q1 * s1 - (int)g.pad[1] + k1 * (int)g.dil[1],
                      i2 = q2 * s2 - (int)g.pad[2] + k2 * (int)g.dil[2];
            if (live && (unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 && (unsigned)i2 < (unsigned)in2)
              at = (uint32_t)((i0 * in1 + i1) * in2 + i2) * 4u;
          } else {
            const int e0 = q0 + (int)g.pad[0] - k0 * (int)g.dil[0], e1 = q1 + (int)g.pad[1] - k1 * (int)g.dil[1],
                      e2 = q2 + (int)g.pad[2] - k2 * (int)g.dil[2];
            int p0 = e0, p1 = e1, p2 = e2;
            if (kClasses) {
              // (the same for every thread of the block: the remainders decide)
              if ((r0 + (int)g.pad[0] - k0 * (int)g.dil[0]) % s0 != 0 || (r1 + (int)g.pad[1] - k1 * (int)g.dil[1]) % s1 != 0 ||
                  (r2 + (int)g.pad[2] - k2 * (int)g.dil[2]) % s2 != 0)
                continue;
              p0 = e0 / s0, p1 = e1 / s1, p2 = e2 / s2; // (exact; negative stays negative)
              if (tid == 0)
                s_tap[used] = t;
            }
            bool fine = live;
            if (!kUnit && !kClasses) { // strides, every thread for itself
              fine = fine && e0 >= 0 && e1 >= 0 && e2 >= 0 && e0 % s0 == 0 && e1 % s1 == 0 && e2 % s2 == 0;
              p0 = e0 / s0, p1 = e1 / s1, p2 = e2 / s2;
            }
            if (fine && (unsigned)p0 < (unsigned)out0 && (unsigned)p1 < (unsigned)out1 && (unsigned)p2 < (unsigned)out2)
              at = (uint32_t)((p0 * out1 + p1) * out2 + p2) * 4u;
          }
          s_reach[used * threads + tid] = at;
          ++used;
        }
    taps = used;
  }
  // (each thread reads back only what it wrote: no barrier for this table)
  uint32_t reach[kTapBatch];
  bool ok[kTapBatch];
  const auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < kTapBatch; ++j) {
      const uint32_t r = t0 + j < taps ? s_reach[(t0 + j) * threads + tid] : kNoReach;
      ok[j] = r != kNoReach, reach[j] = ok[j] ? r : 0u;
    }
  };
  const bool few = taps <= kTapBatch;
  if (few)
    fetch(0);
  const int C = (int)g.C, O = (int)g.O, Cg = (int)g.Cg, Og = (int)g.Og, outer = (int)g.outer;
  const int channels = kForward ? O : C;   // of the result
  const int sources = kForward ? Cg : Og;  // channels of src that meet one channel of the result
  const int64_t Kg = g.Kg;
  // (channels along blockIdx.y, samples along blockIdx.z: no division per pair)
  for (int c = blockIdx.y; c < channels; c += gridDim.y) {
    const int grp = c / (kForward ? Og : Cg), cl = c - grp * Cg; // (cl: backward)
    for (int o0 = 0; o0 < sources; o0 += held) {
      const int no = sources - o0 < held ? sources - o0 : held;
      __syncthreads(); // the previous weights are done with
      for (int i = tid; i < no * taps; i += threads) {
        const int o = i / taps, t = i - o * taps, tap = kClasses ? s_tap[t] : t;
        const int64_t row = kForward ? c : (int64_t)grp * Og + o0 + o; // the weights' channel out
        float wv = kForward ? w[row * Kg + (int64_t)(o0 + o) * all_taps + tap] : w[row * Kg + cl * all_taps + tap];
        if (take_sign)
          wv = (wv > 0.0f) ? 1.0f : ((wv < 0.0f) ? -1.0f : zero_to);
        s_w[i] = scale ? wv * scale[row] : wv;
      }
      __syncthreads();
      if (!live)
        continue;
      for (int n = blockIdx.z; n < outer; n += gridDim.z) {
        const float *rows = src + ((int64_t)n * (kForward ? C : O) + (int64_t)grp * sources + o0) * L;
        float acc = 0.0f;
        if (few) {
          if (taps == kTapBatch)
            for (int o = 0; o < no; o += kOB)
              acc = conv_direct_gather_batch<kOB, kTapBatch, true, kForward>(rows + o * L, L, s_w + o * taps, taps,
                                                                             no - o, taps, reach, ok, acc);
          else if (taps <= 4 && no >= 4) { // (the classes of a strided input gradient, short kernels: few taps of
            if (taps <= 2)                 // four source channels at a time, so that as many loads are in flight)
              for (int o = 0; o < no; o += 4)
                acc = conv_direct_gather_batch<4, 2, false, kForward>(rows + o * L, L, s_w + o * taps, taps, no - o, taps,
                                                                      reach, ok, acc);
            else
              for (int o = 0; o < no; o += 4)
                acc = conv_direct_gather_batch<4, 4, false, kForward>(rows + o * L, L, s_w + o * taps, taps, no - o, taps,
                                                                      reach, ok, acc);
          } else if (taps <= 4)
            for (int o = 0; o < no; o += kOB)
              acc = conv_direct_gather_batch<kOB, 4, false, kForward>(rows + o * L, L, s_w + o * taps, taps, no - o, taps,
                                                                      reach, ok, acc);
          else
            for (int o = 0; o < no; o += kOB)
              acc = conv_direct_gather_batch<kOB, kTapBatch, false, kForward>(rows + o * L, L, s_w + o * taps, taps,
                                                                              no - o, taps, reach, ok, acc);
        } else {
          for (int t0 = 0; t0 < taps; t0 += kTapBatch) {
            fetch(t0);
            for (int o = 0; o < no; o += kOB)
              acc = conv_direct_gather_batch<kOB, kTapBatch, false, kForward>(rows + o * L, L, s_w + o * taps + t0, taps,
                                                                              no - o, taps - t0, reach, ok, acc);
          }
        }
        float *out = dst + ((int64_t)n * channels + c) * positions + pos;
        if (kForward && bias && o0 + no == sources)
          acc = acc + bias[c];
        *out = (accum || o0 > 0) ? *out + acc : acc;
      }
    }
  }
}

// dW[o, k] (+)= sum over samples and output positions of dy[n, o, p] * x[n, c(k), window(p, tap(k))]; one block per
// weight, 256 interleaved partial sums folded in a fixed order.
__global__ __launch_bounds__(kDirectBlock) void conv_direct_dw(const float *__restrict__ dy, const float *__restrict__ x,
                                                               float *__restrict__ dW, ConvGeom g, int accum) {
  __shared__ float part[kDirectBlock];
  const int64_t ok = blockIdx.x, o = ok / g.Kg, k = ok - o * g.Kg, grp = o / g.Og;
  const int64_t c = k / g.k_size;
  int t = (int)(k - c * g.k_size);
  const int k2 = t % g.k[2];
  t /= g.k[2];
  const int k1 = t % g.k[1], k0 = t / g.k[1];
  float acc = 0.0f;
  const int64_t M = g.outer * g.out_sp_size;
  for (int64_t m = threadIdx.x; m < M; m += kDirectBlock) {
    const int64_t n = m / g.out_sp_size, p = m - n * g.out_sp_size;
    const Position q = out_position(g, p);
    const int i0 = q.o0 * g.stride[0] - g.pad[0] + k0 * g.dil[0], i1 = q.o1 * g.stride[1] - g.pad[1] + k1 * g.dil[1],
              i2 = q.o2 * g.stride[2] - g.pad[2] + k2 * g.dil[2];
    const bool in = (unsigned)i0 < (unsigned)g.in_sp[0] && (unsigned)i1 < (unsigned)g.in_sp[1] &&
                    (unsigned)i2 < (unsigned)g.in_sp[2];
    const float xv =
        in ? x[(n * g.C + grp * g.Cg + c) * g.in_sp_size + ((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2] + i2] : 0.0f;
    acc = acc + dy[(n * g.O + o) * g.out_sp_size + p] * xv;
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int s = kDirectBlock / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s)
      part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0)
    dW[ok] = accum ? dW[ok] + part[0] : part[0];
}

// dW of small groups, a thread per output position: block (kO channels out of one group x one channel in, tile of
// the positions, run of the samples).  A thread keeps its position while it walks the samples, so the window's
// place, the taps' offsets (LDS) and which taps fall into the padding (a bit mask) are found once; per sample and tap
// there is one load of x and kO products with the kO values of dy.  When a tile has fewer than 256 positions the
// block's threads take several samples side by side.  Sums in registers (indexed statically), folded over the block
// at the end; partial results [tile * runs + run][O * Kg].
template <int kO, int kTaps>
__global__ __launch_bounds__(kDirectBlock) void conv_direct_dw_pairs(const float *__restrict__ dy,
                                                                     const float *__restrict__ x,
                                                                     float *__restrict__ partial, ConvGeom g,
                                                                     int lanes_p, int runs, int tap_groups) {
  __shared__ int s_off[kTaps][4];
  __shared__ float s_sum[kDirectBlock / 64][kO * kTaps];
  // (kernels of more taps than the template holds: the taps in groups of kTaps, a block per group)
  const int tap0 = (int)(blockIdx.x % tap_groups) * kTaps, tid = threadIdx.x;
  const int taps = (int)g.k_size - tap0 < kTaps ? (int)g.k_size - tap0 : kTaps;
  if (tid < taps) {
    int t = tap0 + tid;
    const int k2 = t % g.k[2];
    t /= g.k[2];
    const int d0 = (t / g.k[1]) * g.dil[0], d1 = (t % g.k[1]) * g.dil[1], d2 = k2 * g.dil[2];
    s_off[tid][0] = d0, s_off[tid][1] = d1, s_off[tid][2] = d2;
    s_off[tid][3] = (d0 * g.in_sp[1] + d1) * g.in_sp[2] + d2;
  }
  __syncthreads();
  const int64_t og = g.Og / kO; // blocks of channels out per group
  const int64_t pair = blockIdx.x / tap_groups, ob = pair / g.Cg, c = pair - ob * g.Cg, grp = ob / og, o = grp * g.Og + (ob - grp * og) * kO;
  const int sub = tid / lanes_p, nsub = kDirectBlock / lanes_p;
  const int64_t p = (int64_t)blockIdx.y * lanes_p + (tid - sub * lanes_p);
  const int64_t per = ceil_div(g.outer, (int64_t)runs), n0 = (int64_t)blockIdx.z * per,
                n1 = n0 + per < g.outer ? n0 + per : g.outer;
  float acc[kO][kTaps];
#pragma unroll
  for (int j = 0; j < kO; ++j)
#pragma unroll
    for (int t = 0; t < kTaps; ++t)
      acc[j][t] = 0.0f;
  if (p < g.out_sp_size) {
    const Position q = out_position(g, p);
    const int b0 = q.o0 * g.stride[0] - g.pad[0], b1 = q.o1 * g.stride[1] - g.pad[1], b2 = q.o2 * g.stride[2] - g.pad[2];
    // per tap, once: the byte offset into a channel of x, and all ones where the tap lies inside the input (taps in
    // the padding, and the template's taps beyond the kernel's, load the channel's first element and mask it to zero)
    const int in0 = (int)g.in_sp[0], in1 = (int)g.in_sp[1], in2 = (int)g.in_sp[2];
    const int first = (b0 * in1 + b1) * in2 + b2; // (negative in the padding: masked)
    uint32_t off[kTaps], inside = 0;
#pragma unroll
    for (int t = 0; t < kTaps; ++t) {
      off[t] = 0;
      if (t < taps) {
        const int i0 = b0 + s_off[t][0], i1 = b1 + s_off[t][1], i2 = b2 + s_off[t][2];
        if ((unsigned)i0 < (unsigned)in0 && (unsigned)i1 < (unsigned)in1 && (unsigned)i2 < (unsigned)in2)
          inside |= 1u << t, off[t] = (uint32_t)(first + s_off[t][3]) * 4u;
      }
    }
    for (int64_t n = n0 + sub; n < n1; n += nsub) {
      float gy[kO];
#pragma unroll
      for (int j = 0; j < kO; ++j)
        gy[j] = dy[(n * g.O + o + j) * g.out_sp_size + p];
      const char *xc = reinterpret_cast<const char *>(x + (n * g.C + grp * g.Cg + c) * g.in_sp_size);
      float xv[kTaps];
#pragma unroll
      for (int t = 0; t < kTaps; ++t)
        xv[t] = *reinterpret_cast<const float *>(xc + off[t]);
#pragma unroll
      for (int t = 0; t < kTaps; ++t) {
        const uint32_t keep = 0u - ((inside >> t) & 1u);
        const float v = __uint_as_float(__float_as_uint(xv[t]) & keep);
#pragma unroll
        for (int j = 0; j < kO; ++j)
          acc[j][t] = acc[j][t] + gy[j] * v;
      }
    }
  }
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int j = 0; j < kO; ++j)
#pragma unroll
    for (int t = 0; t < kTaps; ++t) {
      if (t < taps) {
        float v = acc[j][t];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1)
          v += __shfl_xor(v, off);
        if (lane == 0)
          s_sum[wave][j * kTaps + t] = v;
      }
    }
  __syncthreads();
  if (tid < kO * kTaps && tid % kTaps < taps) {
    float v = s_sum[0][tid];
    for (int w = 1; w < kDirectBlock / 64; ++w)
      v += s_sum[w][tid];
    const int j = tid / kTaps, t = tid - j * kTaps;
    const int64_t chunk = (int64_t)blockIdx.y * runs + blockIdx.z;
    partial[chunk * g.O * g.Kg + (o + j) * g.Kg + c * g.k_size + tap0 + t] = v;
  }
}
// db likewise: block (o, chunk), partial results [chunk][O]
__global__ __launch_bounds__(kDirectBlock) void conv_direct_db_chunks(const float *__restrict__ dy,
                                                                      float *__restrict__ partial, ConvGeom g,
                                                                      int nchunks) {
  __shared__ float s_sum[kDirectBlock / 64];
  const int64_t o = blockIdx.x, per = ceil_div(g.M, (int64_t)nchunks), m0 = (int64_t)blockIdx.y * per,
                m1 = m0 + per < g.M ? m0 + per : g.M;
  float acc = 0.0f;
  if (g.M < ((int64_t)1 << 31)) { // (the usual case: one 32-bit division per element)
    const uint32_t L = (uint32_t)g.out_sp_size;
    for (uint32_t m = (uint32_t)m0 + threadIdx.x; m < (uint32_t)m1; m += kDirectBlock) {
      const uint32_t n = m / L, p = m - n * L;
      acc = acc + dy[((int64_t)n * g.O + o) * g.out_sp_size + p];
    }
  } else {
    for (int64_t m = m0 + threadIdx.x; m < m1; m += kDirectBlock) {
      const int64_t n = m / g.out_sp_size, p = m - n * g.out_sp_size;
      acc = acc + dy[(n * g.O + o) * g.out_sp_size + p];
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    acc += __shfl_xor(acc, off);
  if ((threadIdx.x & 63) == 0)
    s_sum[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0)
    partial[(int64_t)blockIdx.y * g.O + o] = ((s_sum[0] + s_sum[1]) + s_sum[2]) + s_sum[3];
}

// dW for few weights under many windows (the first layers of an image network: 64 x 147 or 64 x 576 weights, 10^5
// windows and more), where the digit operands of the matrix-core product cost more than the product: a block owns a
// tile of 64 output channels x 64 columns k of one group and a run of windows, stages 32 windows at a time in LDS
// (dy as [channel][window], the unfolded input as [k][window], gathered straight from x) and a thread accumulates
// 4 x 4 weights in registers; the runs' partial results [chunk][O * Kg] are added up in chunk order afterwards.
constexpr int kDwTile = 64, kDwWin = 32, kDwPitch = kDwWin + 1;
__global__ __launch_bounds__(kDirectBlock) void conv_direct_dw_tile(const float *__restrict__ dy,
                                                                    const float *__restrict__ x,
                                                                    float *__restrict__ partial, ConvGeom g,
                                                                    int64_t ktiles, int64_t otiles, int nchunks) {
  __shared__ float s_dy[kDwTile * kDwPitch], s_col[kDwTile * kDwPitch];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  int64_t b = blockIdx.x;
  const int64_t kt = b % ktiles;
  b /= ktiles;
  const int64_t ot = b % otiles, grp = b / otiles;
  const int64_t o_base = ot * kDwTile, k_base = kt * kDwTile;
  const int64_t per = ceil_div(ceil_div(g.M, (int64_t)nchunks), (int64_t)kDwWin) * kDwWin;
  const int64_t m0 = (int64_t)blockIdx.y * per, m1 = m0 + per < g.M ? m0 + per : g.M;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[i][j] = 0.0f;
  // A thread stages the same window slot w and the same eight rows r = tid / 32 + 8 i of both tiles in every step:
  // the rows' channel and tap offsets are found once, a step only splits its window index.
  constexpr int kStage = (kDwTile * kDwWin) / kDirectBlock;
  const int w = tid & (kDwWin - 1), r0 = tid >> 5;
  int64_t ch_off[kStage];
  int d0[kStage], d1[kStage], d2[kStage];
  bool k_in[kStage], o_in[kStage];
#pragma unroll
  for (int i = 0; i < kStage; ++i) {
    const int64_t k = k_base + r0 + 8 * i;
    k_in[i] = k < g.Kg;
    o_in[i] = o_base + r0 + 8 * i < g.Og;
    int64_t t = k_in[i] ? k : 0;
    const int k2 = (int)(t % g.k[2]);
    t /= g.k[2];
    const int k1 = (int)(t % g.k[1]);
    t /= g.k[1];
    const int k0 = (int)(t % g.k[0]);
    ch_off[i] = (grp * g.Cg + t / g.k[0]) * g.in_sp_size;
    d0[i] = k0 * g.dil[0], d1[i] = k1 * g.dil[1], d2[i] = k2 * g.dil[2];
  }
  for (int64_t ms = m0; ms < m1; ms += kDwWin) {
    const int64_t m = ms + w;
    const bool m_in = m < m1;
    const int64_t n = m_in ? m / g.out_sp_size : 0, p = m_in ? m - n * g.out_sp_size : 0;
    const Position q = out_position(g, p);
    const int b0 = q.o0 * g.stride[0] - g.pad[0], b1 = q.o1 * g.stride[1] - g.pad[1], b2 = q.o2 * g.stride[2] - g.pad[2];
    const float *xn = x + n * g.C * g.in_sp_size;
    const float *dyn = dy + (n * g.O + grp * g.Og + o_base + r0) * g.out_sp_size + p;
#pragma unroll
    for (int i = 0; i < kStage; ++i) {
      const int r = r0 + 8 * i;
      s_dy[r * kDwPitch + w] = (m_in && o_in[i]) ? dyn[(int64_t)8 * i * g.out_sp_size] : 0.0f;
      const int i0 = b0 + d0[i], i1 = b1 + d1[i], i2 = b2 + d2[i];
      const bool in = m_in && k_in[i] && (unsigned)i0 < (unsigned)g.in_sp[0] && (unsigned)i1 < (unsigned)g.in_sp[1] &&
                      (unsigned)i2 < (unsigned)g.in_sp[2];
      s_col[r * kDwPitch + w] = in ? xn[ch_off[i] + ((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2] + i2] : 0.0f;
    }
    __syncthreads();
#pragma unroll 4
    for (int ww = 0; ww < kDwWin; ++ww) {
      float a[4], c[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = s_dy[(ty * 4 + i) * kDwPitch + ww];
        c[i] = s_col[(tx * 4 + i) * kDwPitch + ww];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = acc[i][j] + a[i] * c[j];
    }
    __syncthreads();
  }
  float *out = partial + (int64_t)blockIdx.y * g.O * g.Kg;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t o = o_base + ty * 4 + i, k = k_base + tx * 4 + j;
      if (o < g.Og && k < g.Kg)
        out[(grp * g.Og + o) * g.Kg + k] = acc[i][j];
    }
}
__global__ __launch_bounds__(kDirectBlock) void conv_direct_dw_final(const float *__restrict__ partial, int nchunks,
                                                                     float *__restrict__ dW, int64_t count, int accum) {
  const int64_t i = (int64_t)blockIdx.x * kDirectBlock + threadIdx.x;
  if (i >= count)
    return;
  float acc = 0.0f;
  for (int c = 0; c < nchunks; ++c)
    acc += partial[(int64_t)c * count + i];
  dW[i] = accum ? dW[i] + acc : acc;
}

// db[o] (+)= sum over samples and positions of dy[n, o, p]
__global__ __launch_bounds__(kDirectBlock) void conv_direct_db(const float *__restrict__ dy, float *__restrict__ db,
                                                               ConvGeom g, int accum) {
  __shared__ float part[kDirectBlock];
  const int64_t o = blockIdx.x, M = g.outer * g.out_sp_size;
  float acc = 0.0f;
  for (int64_t m = threadIdx.x; m < M; m += kDirectBlock) {
    const int64_t n = m / g.out_sp_size, p = m - n * g.out_sp_size;
    acc = acc + dy[(n * g.O + o) * g.out_sp_size + p];
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int s = kDirectBlock / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s)
      part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0)
    db[o] = accum ? db[o] + part[0] : part[0];
}

// Wb = Sign(W) (sign.hpp:48-50) and alpha[o] = (sum of |W[o, :]|) * ((float)1 / Kg)
// (binary_weight_convolution.cpp:66,85-98) for all output channels of all groups: a wavefront per channel, lanes
// along the row, the lanes' sums folded in a fixed order.
__global__ __launch_bounds__(kDirectBlock) void binarize_channels(const float *__restrict__ W, float *__restrict__ Wb,
                                                                  float *__restrict__ alpha, int64_t O, int64_t Kg,
                                                                  float zero_to, float inv_k) {
  const int lane = threadIdx.x & 63;
  const int64_t o = (int64_t)blockIdx.x * (kDirectBlock / 64) + (threadIdx.x >> 6);
  if (o >= O)
    return;
  float acc = 0.0f;
  for (int64_t k = lane; k < Kg; k += 64) {
    const float v = W[o * Kg + k];
    Wb[o * Kg + k] = (v > 0.0f) ? 1.0f : ((v < 0.0f) ? -1.0f : zero_to);
    acc += fabsf(v);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    acc += __shfl_xor(acc, off);
  if (alpha && lane == 0)
    alpha[o] = acc * inv_k;
}

unsigned blocks_for(int64_t n) {
  int64_t b = (n + kDirectBlock - 1) / kDirectBlock;
  return (unsigned)(b > 262144 ? 262144 : (b < 1 ? 1 : b));
}

} // namespace

// What the gather kernel's 32-bit arithmetic and its tables in LDS hold.
static bool conv_direct_gather_fits(const ConvGeom &g) {
  return g.k_size <= 128 && g.C <= 0x7fffffff && g.O <= 0x7fffffff && g.outer <= 0x7fffffff &&
         g.in_sp_size < ((int64_t)1 << 30) && g.out_sp_size < ((int64_t)1 << 30);
}

// Groups too small to pay for the general path's launches: its cost is about 25 us of launches per group forward (85
// backward) plus the product at matrix-core rates; this path's, the product at about 10 TFLOP/s of vector fp32.
bool conv_direct_applies(const ConvGeom &g) {
  if (g.group < 2 || g.O * g.Kg > 0x7fffffffll || !conv_direct_gather_fits(g)) // (the backward has no other form here)
    return false;
  const double flops = 2.0 * (double)g.M * (double)g.Kg * (double)g.O;
  return flops / 1e7 < 25.0 * (double)g.group + flops / 1e8;
}
// Output channels per thread of the tiled kernel, or 0 where it does not apply
// (65535: the second grid extent; the tile's weights have to fit the LDS the kernel may use without asking)
static int direct_tile_width(const ConvGeom &g) {
  if (g.Og % 16 == 0 && g.out_sp_size >= 64 && g.outer * (g.O / 16) <= 65535 && g.Kg * 16 <= kDirectLdsFloats)
    return 16;
  if (g.Og % 8 == 0 && g.out_sp_size >= 64 && g.outer * (g.O / 8) <= 65535 && g.Kg * 8 <= kDirectLdsFloats)
    return 8;
  return 0;
}

// The forward alone also for a single group of very few input channels under a kernel of many taps (the first layer
// of an image network: 3 channels, 7 x 7): rows of the unfolded matrix that are mostly padding of the k tiles, which
// the products on the matrix cores gather element by element.
bool conv_direct_forward_applies(const ConvGeom &g) {
  if (conv_direct_applies(g))
    return true;
  if (g.group == 1 && g.Cg <= 4 && g.k_size >= 9 && g.O % 8 == 0 && g.O * g.Kg <= 0x7fffffffll &&
      g.outer * (g.O / 8) <= 0x7fffffffll)
    return true;
  // ... and for at most 64 output channels over fewer than 24 input channels: the matrix-core products work on tiles
  // 256 channels wide and gather such inputs element by element, the tiled fp32 kernel is the faster one
  // ([4,16,16,56,56] x [32,16,3,3,3]: 0.86 ms binary, 0.24 ms real-weight on the matrix cores)
  return g.group == 1 && g.Cg < 24 && g.O <= 64 && direct_tile_width(g) != 0;
}

namespace {

// How conv_direct_dw_pairs would be launched for a geometry.
struct PairsPlan {
  int kO, lanes_p, tap_groups, taps;
  int64_t pairs, tiles, runs;
  bool fits;
  int64_t loads_per_window() const { return pairs * tap_groups * (kO + taps); } // (dy and the taps of x)
};

PairsPlan plan_dw_pairs(const ConvGeom &g, size_t scratch_bytes) {
  PairsPlan p;
  const int64_t floats = (int64_t)(scratch_bytes / sizeof(float)), count = g.O * g.Kg, L = g.out_sp_size;
  // positions per tile: the multiple of 64 that holds them all, 256 at most; the samples share the rest of the block
  p.lanes_p = L > 128 ? 256 : L > 64 ? 128 : 64;
  p.tiles = ceil_div(L, (int64_t)p.lanes_p);
  p.kO = g.k_size <= 9 && g.Og % 4 == 0 ? 4 : g.k_size <= 16 && g.Og % 2 == 0 ? 2 : 1;
  p.pairs = g.O / p.kO * g.Cg;
  // runs of the samples: enough blocks for the chip, each thread with a few samples at least
  p.runs = ceil_div((int64_t)4096, p.pairs * p.tiles);
  const int64_t steps = ceil_div(g.outer, (int64_t)(kDirectBlock / p.lanes_p));
  if (p.runs > steps / 8)
    p.runs = steps / 8;
  if (p.runs < 1)
    p.runs = 1;
  if (p.runs > g.outer)
    p.runs = g.outer;
  p.tap_groups = p.kO == 1 ? (int)ceil_div(g.k_size, (int64_t)32) : 1;
  p.taps = (int)(g.k_size < 32 ? g.k_size : 32);
  p.fits = p.tiles * p.runs * count <= floats && p.pairs * p.tap_groups <= 0x7fffffff && p.tiles <= 65535 &&
           p.runs <= 65535 && g.in_sp_size < ((int64_t)1 << 30);
  return p;
}

int launch_dw_pairs(const float *dy, const float *x, float *dW, const ConvGeom &g, bool accum, float *scratch,
                    const PairsPlan &p, hipStream_t stream) {
  const int64_t count = g.O * g.Kg;
  const dim3 grid((unsigned)(p.pairs * p.tap_groups), (unsigned)p.tiles, (unsigned)p.runs);
  if (p.kO == 4)
    hipLaunchKernelGGL((conv_direct_dw_pairs<4, 9>), grid, dim3(kDirectBlock), 0, stream, dy, x, scratch, g, p.lanes_p,
                       (int)p.runs, 1);
  else if (p.kO == 2)
    hipLaunchKernelGGL((conv_direct_dw_pairs<2, 16>), grid, dim3(kDirectBlock), 0, stream, dy, x, scratch, g, p.lanes_p,
                       (int)p.runs, 1);
  else if (g.k_size <= 9)
    hipLaunchKernelGGL((conv_direct_dw_pairs<1, 9>), grid, dim3(kDirectBlock), 0, stream, dy, x, scratch, g, p.lanes_p,
                       (int)p.runs, 1);
  else
    hipLaunchKernelGGL((conv_direct_dw_pairs<1, 32>), grid, dim3(kDirectBlock), 0, stream, dy, x, scratch, g, p.lanes_p,
                       (int)p.runs, p.tap_groups);
  NBLA_HIP_LAUNCH_CHECK("conv_direct_dw_pairs");
  hipLaunchKernelGGL(conv_direct_dw_final, dim3((unsigned)ceil_div(count, kDirectBlock)), dim3(kDirectBlock), 0, stream,
                     scratch, (int)(p.tiles * p.runs), dW, count, accum ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("conv_direct_dw_final");
  return NBLA_HIP_OK;
}

} // namespace

// Few weights under many windows (see conv_direct_dw_tile); the partial results need chunks * O * Kg floats.
bool conv_direct_dw_applies(const ConvGeom &g) {
  return !conv_direct_applies(g) && g.Og * g.Kg <= 16384 && g.M >= 16384 && g.O * g.Kg <= 0x7fffffffll;
}
static int dw_chunks(const ConvGeom &g) {
  const int64_t tiles = ceil_div(g.Og, kDwTile) * ceil_div(g.Kg, kDwTile) * g.group;
  int64_t chunks = ceil_div(1024, tiles);
  const int64_t most = g.M / (8 * kDwWin); // eight steps per block at least
  if (chunks > most)
    chunks = most;
  if (chunks > g.M / g.O) // the caller's scratch is the unfolded matrix's: M * Kg floats
    chunks = g.M / g.O;
  return (int)(chunks < 1 ? 1 : chunks);
}
int launch_conv_direct_dw(const float *dy, const float *x, float *dW, const ConvGeom &g, bool accum, void *scratch,
                          size_t scratch_bytes, hipStream_t stream) {
  const int chunks = dw_chunks(g);
  if (scratch_bytes < (size_t)chunks * g.O * g.Kg * sizeof(float) || !aligned16(scratch))
    return fail(NBLA_HIP_ERR_MEMORY, "weight gradient: scratch too small or misaligned.");
  const int64_t ktiles = ceil_div(g.Kg, kDwTile), otiles = ceil_div(g.Og, kDwTile);
  // very few weights (a first layer of 3 x 3 taps, 16 or 32 channels): a tile of 64 x 64 would be mostly empty, the
  // kernel that keeps (channel pair, taps) sums per thread loads less (rough counts of loads per window)
  const PairsPlan pairs = plan_dw_pairs(g, scratch_bytes);
  if (pairs.fits && pairs.loads_per_window() < ktiles * otiles * g.group * 1024)
    return launch_dw_pairs(dy, x, dW, g, accum, static_cast<float *>(scratch), pairs, stream);
  float *partial = static_cast<float *>(scratch);
  hipLaunchKernelGGL(conv_direct_dw_tile, dim3((unsigned)(ktiles * otiles * g.group), (unsigned)chunks),
                     dim3(kDirectBlock), 0, stream, dy, x, partial, g, ktiles, otiles, chunks);
  NBLA_HIP_LAUNCH_CHECK("conv_direct_dw_tile");
  const int64_t count = g.O * g.Kg;
  hipLaunchKernelGGL(conv_direct_dw_final, dim3((unsigned)ceil_div(count, kDirectBlock)), dim3(kDirectBlock), 0, stream,
                     partial, chunks, dW, count, accum ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("conv_direct_dw_final");
  return NBLA_HIP_OK;
}

int launch_conv_direct_binarize(const float *W, float *Wb, float *alpha, const ConvGeom &g, float zero_to,
                                hipStream_t stream) {
  hipLaunchKernelGGL(binarize_channels, dim3((unsigned)ceil_div(g.O, kDirectBlock / 64)), dim3(kDirectBlock), 0, stream,
                     W, Wb, alpha, g.O, g.Kg, zero_to, (float)1 / g.Kg);
  NBLA_HIP_LAUNCH_CHECK("binarize_channels");
  return NBLA_HIP_OK;
}

int launch_conv_direct_gather(bool forward, const float *src, const float *w, const float *scale, const float *bias,
                              float *dst, const ConvGeom &g, bool accum, bool take_sign, float zero_to,
                              hipStream_t stream) {
  const bool unit = g.stride[0] == 1 && g.stride[1] == 1 && g.stride[2] == 1;
  // (a strided input gradient: blocks per class of remainders modulo the strides, the largest class sizes the tiles)
  // (with fewer than four source channels the saving does not pay for the smaller blocks and the strided stores)
  const int64_t classes = forward || unit || g.Og < 4 ? 1 : (int64_t)g.stride[0] * g.stride[1] * g.stride[2];
  int64_t positions = forward ? g.out_sp_size : g.in_sp_size;
  if (classes > 1)
    positions = ceil_div((int64_t)g.in_sp[0], (int64_t)g.stride[0]) * ceil_div((int64_t)g.in_sp[1], (int64_t)g.stride[1]) *
                ceil_div((int64_t)g.in_sp[2], (int64_t)g.stride[2]);
  const int64_t channels = forward ? g.O : g.C, sources = forward ? g.Cg : g.Og;
  int threads = positions <= 64 ? 64 : positions <= 128 ? 128 : kDirectBlock; // small channels
  while (threads > 64 && g.k_size * threads > 8192) // the taps' table: 32 KB of LDS at most
    threads /= 2;
  // the weights that meet one channel of the result, `held` source channels at a time: 31 KB more at most (the list of
  // the taps a class uses follows; 64 KB is what a kernel may use without asking)
  const int held = (int)(sources * g.k_size <= 7936 ? sources : 7936 / g.k_size);
  // a block keeps its positions and walks (sample, channel) pairs: about 2048 blocks, the tables used several times
  const int64_t tiles = ceil_div(positions, (int64_t)threads) * classes;
  if (tiles > 0x7fffffff)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution: too many tiles of positions for one launch.");
  int64_t cw = ceil_div((int64_t)2048, tiles);
  if (cw > channels)
    cw = channels;
  if (cw > 65535)
    cw = 65535;
  int64_t nw = ceil_div((int64_t)2048, tiles * cw);
  if (nw > g.outer)
    nw = g.outer;
  if (nw > 65535)
    nw = 65535;
  const dim3 grid((unsigned)tiles, (unsigned)cw, (unsigned)nw);
  const size_t lds = ((size_t)g.k_size * threads + (size_t)held * g.k_size + (size_t)g.k_size) * sizeof(uint32_t);
#define NBLA_CONV_DIRECT_GATHER(kForward, kUnit, kClasses)                                                              \
  hipLaunchKernelGGL((conv_direct_gather<kForward, kUnit, kClasses>), grid, dim3(threads), lds, stream, src, w, scale,  \
                     bias, dst, g, held, accum ? 1 : 0, take_sign ? 1 : 0, zero_to)
  if (forward)
    NBLA_CONV_DIRECT_GATHER(true, true, false);
  else if (unit)
    NBLA_CONV_DIRECT_GATHER(false, true, false);
  else if (classes > 1)
    NBLA_CONV_DIRECT_GATHER(false, false, true);
  else
    NBLA_CONV_DIRECT_GATHER(false, false, false);
#undef NBLA_CONV_DIRECT_GATHER
  NBLA_HIP_LAUNCH_CHECK("conv_direct_gather");
  return NBLA_HIP_OK;
}

// The geometry of the convolution that computes g's input gradient (unit strides): dy in the place of x, the
// channels' roles exchanged, the padding that is left of the kernel's reach.
static bool direct_transposed_geom(const ConvGeom &g, ConvGeom &t) {
  t = g;
  for (int i = 0; i < kMaxSpatial; ++i) {
    if (g.stride[i] != 1)
      return false;
    t.pad[i] = (g.k[i] - 1) * g.dil[i] - g.pad[i];
    if (t.pad[i] < 0)
      return false;
    t.in_sp[i] = g.out_sp[i], t.out_sp[i] = g.in_sp[i];
  }
  t.C = g.O, t.O = g.C, t.Cg = g.Og, t.Og = g.Cg;
  t.in_sp_size = g.out_sp_size, t.out_sp_size = g.in_sp_size;
  t.Kg = t.Cg * g.k_size;
  t.M = g.outer * t.out_sp_size;
  return true;
}

int launch_conv_direct_forward(const float *x, const float *w, const float *scale, const float *bias, float *y,
                               const ConvGeom &g, hipStream_t stream) {
  const int width = direct_tile_width(g);
  if (width == 16) {
    const dim3 grid((unsigned)ceil_div(g.out_sp_size, kDirectBlock), (unsigned)(g.outer * (g.O / 16)));
    hipLaunchKernelGGL((conv_direct_forward_tile<16, false>), grid, dim3(kDirectBlock),
                       (size_t)g.Kg * 16 * sizeof(float), stream, x, w, scale, bias, y, g, 0);
  } else if (width == 8) {
    const dim3 grid((unsigned)ceil_div(g.out_sp_size, kDirectBlock), (unsigned)(g.outer * (g.O / 8)));
    hipLaunchKernelGGL((conv_direct_forward_tile<8, false>), grid, dim3(kDirectBlock), (size_t)g.Kg * 8 * sizeof(float),
                       stream, x, w, scale, bias, y, g, 0);
  } else if (conv_direct_gather_fits(g)) {
    return launch_conv_direct_gather(true, x, w, scale, bias, y, g, false, false, 0.0f, stream);
  } else {
    hipLaunchKernelGGL(conv_direct_forward, dim3(blocks_for(g.outer * g.O * g.out_sp_size)), dim3(kDirectBlock), 0,
                       stream, x, w, scale, bias, y, g);
  }
  NBLA_HIP_LAUNCH_CHECK("conv_direct_forward");
  return NBLA_HIP_OK;
}

// db[o] (+)= sum over samples and positions of dy[n, o, p], every group at once, straight from dy: chunks of the
// windows over blocks (partial sums in the scratch memory, added in a fixed order) where the channels alone would not
// fill the chip.
int launch_conv_direct_db(const float *dy, float *db, const ConvGeom &g, bool accum, float *scratch,
                          size_t scratch_bytes, hipStream_t stream) {
  int64_t chunks = ceil_div((int64_t)4096, g.O);
  if (chunks > g.M / 1024)
    chunks = g.M / 1024;
  if (chunks > (int64_t)(scratch_bytes / sizeof(float)) / g.O)
    chunks = (int64_t)(scratch_bytes / sizeof(float)) / g.O;
  if (chunks > 65535)
    chunks = 65535;
  if (g.O > 0x7fffffff)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution backward: 2^31 channels or more.");
  if (scratch && chunks >= 2) {
    hipLaunchKernelGGL(conv_direct_db_chunks, dim3((unsigned)g.O, (unsigned)chunks), dim3(kDirectBlock), 0, stream, dy,
                       scratch, g, (int)chunks);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_db_chunks");
    hipLaunchKernelGGL(conv_direct_dw_final, dim3((unsigned)ceil_div(g.O, kDirectBlock)), dim3(kDirectBlock), 0, stream,
                       scratch, (int)chunks, db, g.O, accum ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_dw_final");
  } else {
    hipLaunchKernelGGL(conv_direct_db, dim3((unsigned)g.O), dim3(kDirectBlock), 0, stream, dy, db, g, accum ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_db");
  }
  return NBLA_HIP_OK;
}

// The input gradient in the direct forms: through the tiled kernel where a group has 8 or 16 input channels to share
// (unit strides), as a gather otherwise.
int launch_conv_direct_dx(const float *dy, const float *w, const float *scale, float *dx, const ConvGeom &g, bool accum,
                          bool take_sign, float zero_to, float *scratch, size_t scratch_bytes, hipStream_t stream) {
  ConvGeom t;
  const int width = scratch && direct_transposed_geom(g, t) && (size_t)(g.O * g.Kg) * sizeof(float) <= scratch_bytes
                        ? direct_tile_width(t)
                        : 0;
  if (width) {
    // channels to share: the input gradient as a convolution of dy with the transposed, reversed weights (in the
    // scratch memory, which is free again when the launch has run)
    const int64_t count = g.O * g.Kg;
    hipLaunchKernelGGL(conv_direct_transpose_weights, dim3((unsigned)ceil_div(count, kDirectBlock)), dim3(kDirectBlock),
                       0, stream, w, scale, scratch, count, (int)g.Og, (int)g.Cg, (int)g.k_size, take_sign ? 1 : 0,
                       zero_to);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_transpose_weights");
    const dim3 grid((unsigned)ceil_div(t.out_sp_size, kDirectBlock), (unsigned)(t.outer * (t.O / width)));
    const size_t lds = (size_t)(t.Kg + 1) * width * sizeof(float);
    if (width == 16)
      hipLaunchKernelGGL((conv_direct_forward_tile<16, true>), grid, dim3(kDirectBlock), lds, stream, dy, scratch,
                         nullptr, nullptr, dx, t, accum ? 1 : 0);
    else
      hipLaunchKernelGGL((conv_direct_forward_tile<8, true>), grid, dim3(kDirectBlock), lds, stream, dy, scratch,
                         nullptr, nullptr, dx, t, accum ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_forward_tile");
    return NBLA_HIP_OK;
  }
  if (!conv_direct_gather_fits(g))
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution backward: more than 128 taps, 2^31 channels or samples, "
                                              "or 2^30 positions per channel, in the direct form.");
  return launch_conv_direct_gather(false, dy, w, scale, nullptr, dx, g, accum, take_sign, zero_to, stream);
}

// The input gradient of a single group of at most four input channels (a network's first layer) as a gather, where
// that is little work: the general path unfolds the gradient for every input position and folds it back.
bool conv_direct_dx_applies(const ConvGeom &g) {
  return g.group == 1 && g.Cg <= 4 && conv_direct_gather_fits(g) &&
         (double)g.outer * (double)g.in_sp_size * (double)g.Cg * (double)g.O * (double)g.k_size < 2.5e8;
}

int launch_conv_direct_backward(const float *dy, const float *x, const float *w, const float *scale, float *dx,
                                float *dW, float *db, const ConvGeom &g, bool accum_x, bool accum_w, bool accum_b,
                                bool take_sign, float zero_to, float *scratch, size_t scratch_bytes,
                                hipStream_t stream) {
  if (dx) {
    const int rc =
        launch_conv_direct_dx(dy, w, scale, dx, g, accum_x, take_sign, zero_to, scratch, scratch_bytes, stream);
    if (rc)
      return rc;
  }
  if (dW) { // (after dx in the stream: the scratch memory is free again)
    const PairsPlan p = plan_dw_pairs(g, scratch_bytes);
    if (scratch && p.fits) {
      const int rc = launch_dw_pairs(dy, x, dW, g, accum_w, scratch, p, stream);
      if (rc)
        return rc;
    } else {
      hipLaunchKernelGGL(conv_direct_dw, dim3((unsigned)(g.O * g.Kg)), dim3(kDirectBlock), 0, stream, dy, x, dW, g,
                         accum_w ? 1 : 0);
      NBLA_HIP_LAUNCH_CHECK("conv_direct_dw");
    }
  }
  if (db) // (after dW's final sum in the stream)
    return launch_conv_direct_db(dy, db, g, accum_b, scratch, scratch_bytes, stream);
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
