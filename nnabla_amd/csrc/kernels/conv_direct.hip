// Grouped convolutions with small groups (depthwise, ResNeXt-style): every group's product is far too small for the
// matrix cores, and the general path pays several launches per group (256 groups of a depthwise layer: milliseconds
// of launches around microseconds of work).  These kernels compute all groups in one launch each, in plain fp32 with
// one thread per output element and the contraction in the reference's order k = (channel, tap)
// (convolution.cpp:161-197 forward, :199-330 backward: per sample and group an unfold and a product -- here without
// the unfolded matrix).  The same kernels serve the binary convolutions: the weights are then the materialised signs,
// multiplied by alpha[o] as binary_weight_convolution.cpp:100-110 forms Ws.
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
template <int kOut>
__global__ __launch_bounds__(kDirectBlock) void conv_direct_forward_tile(const float *__restrict__ x,
                                                                         const float *__restrict__ w,
                                                                         const float *__restrict__ scale,
                                                                         const float *__restrict__ bias,
                                                                         float *__restrict__ y, ConvGeom g) {
  extern __shared__ __attribute__((aligned(16))) float s_w[]; // [Kg][kOut]
  typedef float float4_d __attribute__((ext_vector_type(4)));
  const int64_t otiles = g.O / kOut;
  const int64_t n = blockIdx.y / otiles, o0 = (blockIdx.y - n * otiles) * kOut, grp = o0 / g.Og;
  const int Kg = (int)g.Kg;
  for (int i = threadIdx.x; i < Kg * kOut; i += kDirectBlock) {
    const int j = i / Kg, k = i - j * Kg; // consecutive threads read consecutive k of one channel
    const float wv = w[(o0 + j) * g.Kg + k];
    s_w[k * kOut + j] = scale ? wv * scale[o0 + j] : wv; // Ws = Wb * alpha, rounded once as the reference forms it
  }
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
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int i2 = b2 + (k2 + u) * g.dil[2];
            xv[u] = (row_in && k2 + u < g.k[2] && (unsigned)i2 < (unsigned)g.in_sp[2]) ? xr[i2] : 0.0f;
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            if (k2 + u < g.k[2]) { // uniform
              const float4_d *wk = reinterpret_cast<const float4_d *>(s_w + (t + u) * kOut);
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
      y[(n * g.O + o0 + j) * g.out_sp_size + p] = bias ? acc[j] + bias[o0 + j] : acc[j];
  }
}

// dx[n, c, q] (+)= sum over the group's o and the taps whose window position p lies in the output:
// (dy[n, o, p] * scale[o]) * w[o, c, tap]   (the unfolded gradient folded back, convolution.cpp:262-283)
// take_sign: w holds the real-valued weights of a binary convolution, whose signs (sign.hpp:48-50) are what the
// forward pass multiplied with.
__global__ __launch_bounds__(kDirectBlock) void conv_direct_dx(const float *__restrict__ dy, const float *__restrict__ w,
                                                               const float *__restrict__ scale, float *__restrict__ dx,
                                                               ConvGeom g, int accum, int take_sign, float zero_to) {
  const int64_t total = g.outer * g.C * g.in_sp_size;
  for (int64_t i = (int64_t)blockIdx.x * kDirectBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kDirectBlock) {
    int64_t pos = i % g.in_sp_size;
    const int64_t nc = i / g.in_sp_size, c = nc % g.C, n = nc / g.C, grp = c / g.Cg, cl = c - grp * g.Cg;
    const int q2 = (int)(pos % g.in_sp[2]);
    pos /= g.in_sp[2];
    const int q1 = (int)(pos % g.in_sp[1]), q0 = (int)(pos / g.in_sp[1]);
    const float *dyn = dy + (n * g.O + grp * g.Og) * g.out_sp_size;
    const float *wg = w + (grp * g.Og) * g.Kg + cl * g.k_size;
    float acc = 0.0f;
    int t = 0;
    for (int k0 = 0; k0 < g.k[0]; ++k0)
      for (int k1 = 0; k1 < g.k[1]; ++k1)
        for (int k2 = 0; k2 < g.k[2]; ++k2, ++t) {
          const int e0 = q0 + g.pad[0] - k0 * g.dil[0], e1 = q1 + g.pad[1] - k1 * g.dil[1],
                    e2 = q2 + g.pad[2] - k2 * g.dil[2];
          if (e0 < 0 || e1 < 0 || e2 < 0 || e0 % g.stride[0] || e1 % g.stride[1] || e2 % g.stride[2])
            continue;
          const int p0 = e0 / g.stride[0], p1 = e1 / g.stride[1], p2 = e2 / g.stride[2];
          if (p0 >= g.out_sp[0] || p1 >= g.out_sp[1] || p2 >= g.out_sp[2])
            continue;
          const int64_t p = ((int64_t)p0 * g.out_sp[1] + p1) * g.out_sp[2] + p2;
          for (int64_t o = 0; o < g.Og; ++o) {
            const float gy = dyn[o * g.out_sp_size + p];
            const float gs = scale ? gy * scale[grp * g.Og + o] : gy;
            float wv = wg[o * g.Kg + t];
            if (take_sign)
              wv = (wv > 0.0f) ? 1.0f : ((wv < 0.0f) ? -1.0f : zero_to);
            acc = acc + gs * wv;
          }
        }
    dx[i] = accum ? dx[i] + acc : acc;
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

// Groups too small to pay for the general path's launches: its cost is about 25 us of launches per group forward (85
// backward) plus the product at matrix-core rates; this path's, the product at about 10 TFLOP/s of vector fp32.
bool conv_direct_applies(const ConvGeom &g) {
  if (g.group < 2 || g.O * g.Kg > 0x7fffffffll)
    return false;
  const double flops = 2.0 * (double)g.M * (double)g.Kg * (double)g.O;
  return flops / 1e7 < 25.0 * (double)g.group + flops / 1e8;
}
// The forward alone also for a single group of very few input channels under a kernel of many taps (the first layer
// of an image network: 3 channels, 7 x 7): rows of the unfolded matrix that are mostly padding of the k tiles, which
// the products on the matrix cores gather element by element.
bool conv_direct_forward_applies(const ConvGeom &g) {
  if (conv_direct_applies(g))
    return true;
  return g.group == 1 && g.Cg <= 4 && g.k_size >= 9 && g.O % 8 == 0 && g.O * g.Kg <= 0x7fffffffll &&
         g.outer * (g.O / 8) <= 0x7fffffffll;
}

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

int launch_conv_direct_forward(const float *x, const float *w, const float *scale, const float *bias, float *y,
                               const ConvGeom &g, hipStream_t stream) {
  // (65535: the second grid extent; the tile's weights have to fit the LDS the kernel may use without asking)
  if (g.Og % 16 == 0 && g.out_sp_size >= 64 && g.outer * (g.O / 16) <= 65535 && g.Kg * 16 <= kDirectLdsFloats) {
    const dim3 grid((unsigned)ceil_div(g.out_sp_size, kDirectBlock), (unsigned)(g.outer * (g.O / 16)));
    hipLaunchKernelGGL(conv_direct_forward_tile<16>, grid, dim3(kDirectBlock), (size_t)g.Kg * 16 * sizeof(float), stream,
                       x, w, scale, bias, y, g);
  } else if (g.Og % 8 == 0 && g.out_sp_size >= 64 && g.outer * (g.O / 8) <= 65535 && g.Kg * 8 <= kDirectLdsFloats) {
    const dim3 grid((unsigned)ceil_div(g.out_sp_size, kDirectBlock), (unsigned)(g.outer * (g.O / 8)));
    hipLaunchKernelGGL(conv_direct_forward_tile<8>, grid, dim3(kDirectBlock), (size_t)g.Kg * 8 * sizeof(float), stream,
                       x, w, scale, bias, y, g);
  } else {
    hipLaunchKernelGGL(conv_direct_forward, dim3(blocks_for(g.outer * g.O * g.out_sp_size)), dim3(kDirectBlock), 0,
                       stream, x, w, scale, bias, y, g);
  }
  NBLA_HIP_LAUNCH_CHECK("conv_direct_forward");
  return NBLA_HIP_OK;
}

int launch_conv_direct_backward(const float *dy, const float *x, const float *w, const float *scale, float *dx,
                                float *dW, float *db, const ConvGeom &g, bool accum_x, bool accum_w, bool accum_b,
                                bool take_sign, float zero_to, hipStream_t stream) {
  if (dx) {
    hipLaunchKernelGGL(conv_direct_dx, dim3(blocks_for(g.outer * g.C * g.in_sp_size)), dim3(kDirectBlock), 0, stream, dy,
                       w, scale, dx, g, accum_x ? 1 : 0, take_sign ? 1 : 0, zero_to);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_dx");
  }
  if (dW) {
    hipLaunchKernelGGL(conv_direct_dw, dim3((unsigned)(g.O * g.Kg)), dim3(kDirectBlock), 0, stream, dy, x, dW, g,
                       accum_w ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_dw");
  }
  if (db) {
    hipLaunchKernelGGL(conv_direct_db, dim3((unsigned)g.O), dim3(kDirectBlock), 0, stream, dy, db, g, accum_b ? 1 : 0);
    NBLA_HIP_LAUNCH_CHECK("conv_direct_db");
  }
  return NBLA_HIP_OK;
}

} // namespace nbla_hip
