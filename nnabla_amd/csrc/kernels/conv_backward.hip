// Backward passes of the convolutions: Binary{Weight,Connect}Convolution (gradient w.r.t. x on the bit-weight
// product) and Convolution with real-valued weights (INQConvolution), plus weight and bias gradients.
//
// Per group the reference's sample loop (convolution.cpp:199-283) is folded into three matrix products over all
// samples at once, with m = (sample, output position) as the long dimension:
//   dyt [M, Og]          the output gradient of the group, transposed so that m is the row index
//   colg[n][kk][l]       = sum over o of dyt[m, o] * w[o, kk]   (then folded into dx by a gather)
//   dW  [Og, Kg]         = dyt^T . col(x)                        (col(x) [M, Kg] is the unfolded input; digit x digit)
//   db  [O]              = sums of dy over samples and positions, straight from dy
#include "common.hpp"
#include "conv_geom.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

namespace nbla_hip {
namespace {

// dyt[(n * L + l) * Og + o] = dy[(n * O + grp * Og + o) * L + l] * (scale ? scale[o] : 1): a 32 x 32 tile through LDS
// so that both sides move contiguous runs.
__global__ __launch_bounds__(256) void gather_dy(const float *__restrict__ dy, const float *__restrict__ scale,
                                                 float *__restrict__ dyt, int64_t O, int64_t Og, int64_t L,
                                                 int64_t grp) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t n = blockIdx.z, l0 = (int64_t)blockIdx.x * 32, o0 = (int64_t)blockIdx.y * 32;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t o = o0 + ty + 8 * i, l = l0 + tx;
    tile[ty + 8 * i][tx] = (o < Og && l < L) ? dy[(n * O + grp * Og + o) * L + l] : 0.0f;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t l = l0 + ty + 8 * i, o = o0 + tx;
    if (l < L && o < Og) {
      const float v = tile[tx][ty + 8 * i];
      dyt[(n * L + l) * Og + o] = scale ? v * scale[o] : v;
    }
  }
}

// dx element (n, c, position) (+)= sum of the unfolded gradient over the taps that read that position, in
// ascending tap order (the order fold_from_patches.cpp:125-170 adds them in).  colg is [outer][Kg][L].
// One thread per element of a sample's channel group; 32-bit arithmetic inside the sample (the host checks that it
// fits); kUnitStride drops the divisions of the general case.
template <bool kUnitStride>
__global__ __launch_bounds__(256) void col2im_gather(const float *__restrict__ colg, float *__restrict__ dx, ConvGeom g,
                                                     int64_t grp, int accumulate) {
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size, Cg = (int)g.Cg;
  const int out0 = g.out_sp[0], out1 = g.out_sp[1], out2 = g.out_sp[2], L = (int)g.out_sp_size;
  const int K0 = g.k[0], K1 = g.k[1], K2 = g.k[2], taps = (int)g.k_size;
  const int s0 = g.stride[0], s1 = g.stride[1], s2 = g.stride[2];
  const int per_sample = Cg * plane;
  const int64_t n = blockIdx.y;
  const float *sample = colg + n * g.Kg * g.out_sp_size;
  float *dst_sample = dx + (n * g.C + grp * g.Cg) * g.in_sp_size;
  for (int idx = blockIdx.x * 256 + threadIdx.x; idx < per_sample; idx += gridDim.x * 256) {
    int t = idx;
    const int i2 = t % in2;
    t /= in2;
    const int i1 = t % in1;
    t /= in1;
    const int i0 = t % in0;
    const int cc = t / in0;
    const float *src = sample + (int64_t)cc * taps * L;
    float acc = 0.0f;
    for (int k0 = 0; k0 < K0; ++k0) {
      const int t0 = i0 + g.pad[0] - k0 * g.dil[0];
      const int q0 = kUnitStride ? t0 : t0 / s0;
      if (t0 < 0 || (!kUnitStride && t0 - q0 * s0 != 0) || q0 >= out0)
        continue;
      for (int k1 = 0; k1 < K1; ++k1) {
        const int t1 = i1 + g.pad[1] - k1 * g.dil[1];
        const int q1 = kUnitStride ? t1 : t1 / s1;
        if (t1 < 0 || (!kUnitStride && t1 - q1 * s1 != 0) || q1 >= out1)
          continue;
        for (int k2 = 0; k2 < K2; ++k2) {
          const int t2 = i2 + g.pad[2] - k2 * g.dil[2];
          const int q2 = kUnitStride ? t2 : t2 / s2;
          if (t2 < 0 || (!kUnitStride && t2 - q2 * s2 != 0) || q2 >= out2)
            continue;
          const int tap = (k0 * K1 + k1) * K2 + k2;
          acc += src[(int64_t)tap * L + (q0 * out1 + q1) * out2 + q2];
        }
      }
    }
    float *dst = dst_sample + idx;
    *dst = accumulate ? *dst + acc : acc;
  }
}

// The same for unit strides and at most 64 taps, with the loads of sixteen taps in flight at a time (the loop above
// waits for every load before it issues the next: nine round trips to the L2 for a 3 x 3 kernel).  The taps'
// displacements are decoded once per block into LDS; a tap that does not reach the element contributes through a
// select, not through an addition of zero, so the sum is the same chain of additions as above.
__global__ __launch_bounds__(256) void col2im_gather_unit(const float *__restrict__ colg, float *__restrict__ dx,
                                                          ConvGeom g, int64_t grp, int accumulate) {
  typedef int i32x4_t __attribute__((ext_vector_type(4)));
  __shared__ i32x4_t s_taps[64]; // {displacement along each spatial axis, 0}
  const int in0 = g.in_sp[0], in1 = g.in_sp[1], in2 = g.in_sp[2], plane = (int)g.in_sp_size, Cg = (int)g.Cg;
  const int out0 = g.out_sp[0], out1 = g.out_sp[1], out2 = g.out_sp[2], L = (int)g.out_sp_size;
  const int taps = (int)g.k_size;
  if ((int)threadIdx.x < taps) {
    int q = threadIdx.x;
    const int k2 = q % g.k[2];
    q /= g.k[2];
    const int k1 = q % g.k[1], k0 = q / g.k[1];
    s_taps[threadIdx.x] = i32x4_t{k0 * g.dil[0] - g.pad[0], k1 * g.dil[1] - g.pad[1], k2 * g.dil[2] - g.pad[2], 0};
  }
  __syncthreads();
  const int per_sample = Cg * plane;
  const int64_t n = blockIdx.y;
  const float *sample = colg + n * g.Kg * g.out_sp_size;
  float *dst_sample = dx + (n * g.C + grp * g.Cg) * g.in_sp_size;
  for (int idx = blockIdx.x * 256 + threadIdx.x; idx < per_sample; idx += gridDim.x * 256) {
    int t = idx;
    const int i2 = t % in2;
    t /= in2;
    const int i1 = t % in1;
    t /= in1;
    const int i0 = t % in0;
    const int cc = t / in0;
    const float *src = sample + (int64_t)cc * taps * L;
    float acc = 0.0f;
    for (int tap0 = 0; tap0 < taps; tap0 += 16) {
      float v[16];
      bool ok[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int tap = tap0 + j < taps ? tap0 + j : taps - 1;
        const i32x4_t d = s_taps[tap];
        const int q0 = i0 - d.x, q1 = i1 - d.y, q2 = i2 - d.z;
        ok[j] = tap0 + j < taps && (unsigned)q0 < (unsigned)out0 && (unsigned)q1 < (unsigned)out1 &&
                (unsigned)q2 < (unsigned)out2;
        v[j] = src[ok[j] ? tap * L + (q0 * out1 + q1) * out2 + q2 : 0];
      }
#pragma unroll
      for (int j = 0; j < 16; ++j)
        acc = ok[j] ? acc + v[j] : acc;
    }
    float *dst = dst_sample + idx;
    *dst = accumulate ? *dst + acc : acc;
  }
}

struct ConvBackwardPlan {
  size_t dyt_off, col_off, a_planes_off, b_planes_off, digits_off, bits_off, prep_off, count_off,
      flag_off, sums_off, slab_off, total;
};

size_t larger(size_t a, size_t b) { return a > b ? a : b; }

// One layout for both entry points; every region is reused group after group.
ConvBackwardPlan plan_conv_backward(const ConvGeom &g) {
  ConvBackwardPlan p;
  size_t off = 0;
  const size_t dyt_bytes = round_up((size_t)g.M * g.Og * sizeof(float), 256);
  p.dyt_off = off;
  off += dyt_bytes;
  p.col_off = off; // unfolded input [M, Kg], and the unfolded gradient [outer][Kg][L]
  off += round_up((size_t)g.M * g.Kg * sizeof(float), 256);
  p.a_planes_off = off; // dyt^T for dW (rows o, contraction m) or dyt for dx (rows m, contraction o)
  off += round_up(larger(nbla_hip_digit_operand_bytes(g.M, g.Og), nbla_hip_digit_operand_bytes(g.Og, g.M)), 256);
  p.b_planes_off = off; // col(x) (columns kk, contraction m) or w (columns kk, contraction o)
  off += round_up(larger(nbla_hip_digit_operand_bytes(g.Kg, g.M), nbla_hip_digit_operand_bytes(g.Kg, g.Og)), 256);
  p.digits_off = off;
  off += round_up(nbla_hip_digit_operand_bytes(g.M, g.Og), 256);
  p.bits_off = off;
  off += round_up(nbla_hip_packed_bits_bytes(g.Og, g.Kg), 256);
  p.prep_off = off;
  off += round_up(nbla_hip_binarize_workspace_bytes(g.Og, g.Kg), 256);
  p.count_off = off;
  off += 256;
  p.flag_off = off;
  off += 256;
  p.sums_off = off;
  off += round_up(column_sums_workspace_bytes(g.M, g.Og), 256);
  p.slab_off = off; // packed bits of the transposed convolution, when the input gradient takes that form
  {
    ConvGeom t;
    if (conv_slab_transposed_geom(g, t))
      off += round_up(conv_slab_prepared_bytes(t), 256);
  }
  p.total = off;
  return p;
}

int launch_gather_dy(const float *dy, const float *scale, float *dyt, const ConvGeom &g, int64_t grp,
                     hipStream_t stream) {
  if (g.outer > 65535 || ceil_div(g.Og, 32) > 65535)
    return fail(NBLA_HIP_ERR_VALUE, "convolution backward supports at most 65535 samples per call.");
  const dim3 grid((unsigned)ceil_div(g.out_sp_size, 32), (unsigned)ceil_div(g.Og, 32), (unsigned)g.outer);
  hipLaunchKernelGGL(gather_dy, grid, dim3(256), 0, stream, dy, scale, dyt, g.O, g.Og, g.out_sp_size, grp);
  NBLA_HIP_LAUNCH_CHECK("gather_dy");
  return NBLA_HIP_OK;
}

int launch_col2im(const float *colg, float *dx, const ConvGeom &g, int64_t grp, bool accumulate, hipStream_t stream) {
  if (g.Cg * g.in_sp_size >= ((int64_t)1 << 31) || g.k_size * g.out_sp_size >= ((int64_t)1 << 31) || g.outer > 65535)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "convolution backward: a sample's channel group or unfolded channel has "
                                              "2^31 elements or more, or more than 65535 samples.");
  int64_t bx = ceil_div(g.Cg * g.in_sp_size, 256);
  if (bx > 65536)
    bx = 65536;
  const dim3 grid((unsigned)bx, (unsigned)g.outer);
  const bool unit = g.stride[0] == 1 && g.stride[1] == 1 && g.stride[2] == 1;
  if (unit && g.k_size <= 64)
    hipLaunchKernelGGL(col2im_gather_unit, grid, dim3(256), 0, stream, colg, dx, g, grp, accumulate ? 1 : 0);
  else if (unit)
    hipLaunchKernelGGL(col2im_gather<true>, grid, dim3(256), 0, stream, colg, dx, g, grp, accumulate ? 1 : 0);
  else
    hipLaunchKernelGGL(col2im_gather<false>, grid, dim3(256), 0, stream, colg, dx, g, grp, accumulate ? 1 : 0);
  NBLA_HIP_LAUNCH_CHECK("col2im_gather");
  return NBLA_HIP_OK;
}

// `binary`: the weights of the forward pass were Sign(W) (* alpha[o]); otherwise W itself.
int conv_backward(const float *dy, const float *x, const float *W, const float *Wb, const float *alpha, float *dx,
                  float *dW, float *db, const ConvGeom &g, bool binary, float zero_to, bool accum_x, bool accum_w,
                  bool accum_b, void *workspace, size_t workspace_bytes, void *stream_) {
  const ConvBackwardPlan p = plan_conv_backward(g);
  if (workspace_bytes < p.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "convolution backward workspace too small (%zu < %zu) or misaligned.",
                workspace_bytes, p.total);
  int rc = ensure_init();
  if (rc)
    return rc;
  hipStream_t stream = as_stream(stream_);
  if (conv_direct_applies(g)) { // many small groups: all of them in one launch per gradient
    // the forward multiplied with Wb = Sign(W) (* alpha): the signs passed in, or taken from W on the way
    if (binary && !Wb && !(zero_to == 1.0f || zero_to == -1.0f))
      return fail(NBLA_HIP_ERR_VALUE, "the binarised weights are needed when Sign(0) is neither +1 nor -1.");
    return launch_conv_direct_backward(dy, x, (binary && Wb) ? Wb : W, binary ? alpha : nullptr, dx, dW, db, g, accum_x,
                                       accum_w, accum_b, binary && !Wb, zero_to, static_cast<float *>(workspace),
                                       workspace_bytes, stream);
  }
  char *base = static_cast<char *>(workspace);
  float *dyt = reinterpret_cast<float *>(base + p.dyt_off);
  float *col = reinterpret_cast<float *>(base + p.col_off);
  int *count = reinterpret_cast<int *>(base + p.count_off);
  uint32_t *bits = reinterpret_cast<uint32_t *>(base + p.bits_off);
  const bool representable = (zero_to == 1.0f || zero_to == -1.0f);
  const int64_t L = g.out_sp_size;
  // The input gradient of a binary convolution of unit stride is itself a binary convolution (dy in the place of x,
  // channels' roles exchanged, taps flipped): it takes the product that keeps input positions in LDS.
  ConvGeom gt;
  bool dx_slab = dx && binary && representable && conv_slab_transposed_geom(g, gt);
  // a first layer's input gradient (few input channels, little work) as a gather; its scratch memory is the unfolded
  // gradient's buffer, used by the next launches only afterwards in the stream
  if (dx && conv_direct_dx_applies(g) && (!binary || Wb || representable)) {
    rc = launch_conv_direct_dx(dy, (binary && Wb) ? Wb : W, binary ? alpha : nullptr, dx, g, accum_x, binary && !Wb,
                               zero_to, col, (size_t)g.M * g.Kg * sizeof(float), stream);
    if (rc)
      return rc;
    dx = nullptr, dx_slab = false;
  }
  // few weights under many windows: the weight gradient in fp32 straight from dy and x, all groups at once (its
  // partial results lie in the unfolded gradient's buffer, so it runs before the loop that fills that buffer)
  if (dW && conv_direct_dw_applies(g)) {
    rc = launch_conv_direct_dw(dy, x, dW, g, accum_w, col, (size_t)g.M * g.Kg * sizeof(float), stream);
    if (rc)
      return rc;
    dW = nullptr;
  }
  // the bias gradient straight from dy, every group at once (partial sums in the same buffer, after the weight
  // gradient's in the stream)
  if (db) {
    rc = launch_conv_direct_db(dy, db, g, accum_b, col, (size_t)g.M * g.Kg * sizeof(float), stream);
    if (rc)
      return rc;
    db = nullptr;
  }
  for (int64_t grp = 0; grp < g.group; ++grp) {
    const float *Wg = W + grp * g.Og * g.Kg;
    const float *ag = alpha ? alpha + grp * g.Og : nullptr;
    if ((dx && !dx_slab) || dW) {
      rc = launch_gather_dy(dy, nullptr, dyt, g, grp, stream);
      if (rc)
        return rc;
    }
    if (dx_slab) {
      rc = launch_conv_slab_prepare_transposed(Wg, base + p.slab_off, g, zero_to, stream);
      if (rc)
        return rc;
      rc = launch_conv_slab(dy, gt, grp, base + p.slab_off, nullptr, nullptr, nullptr, dx, stream, ag, accum_x);
      if (rc)
        return rc;
    } else if (dx) {
      if (binary) {
        // Sign(W_g) packed for the contraction over o: W_g is stored [Og, Kg] = [contraction][column]
        rc = nbla_hip_binarize_weights_f32(Wg, nullptr, nullptr, bits, g.Og, g.Kg, 0, zero_to,
                                           representable ? nullptr : count, base + p.prep_off,
                                           nbla_hip_binarize_workspace_bytes(g.Og, g.Kg), stream_);
        if (rc)
          return rc;
        rc = nbla_hip_split_digits_scaled_f32(dyt, g.Og, ag, base + p.digits_off, g.M, g.Og, stream_);
        if (rc)
          return rc;
        rc = launch_gemm_bits(base + p.digits_off, bits, nullptr, nullptr, col, g.M, g.Og, g.Kg, L, g.Kg * L, L, true,
                              stream);
        if (rc)
          return rc;
        if (!representable) {
          // Sign(0) is neither +1 nor -1: when the group holds a weight that is neither negative nor positive (counted
          // on the device by the pass above) the unfolded gradient is recomputed in fp32 from the forward's signs,
          //   col[m, kk] = sum_o (dyt[m, o] alpha[o]) Wb[o, kk],
          // by a launch that leaves at once otherwise.  The host never reads the count.
          if (!Wb)
            return fail(NBLA_HIP_ERR_VALUE, "the binarised weights are needed when Sign(0) is neither +1 nor -1.");
          rc = launch_gemm_f32_mapped(dyt, Wb + grp * g.Og * g.Kg, false, nullptr, nullptr, col, g.M, g.Og, g.Kg, L,
                                      g.Kg * L, L, stream, count, ag, false);
        }
      } else {
        // real x real on the digit product: dyt rows m (row-scaled), the weights' columns kk (column-scaled),
        // contraction over the output channels o
        rc = nbla_hip_split_digits_f32(dyt, g.Og, base + p.a_planes_off, g.M, g.Og, stream_);
        if (rc)
          return rc;
        rc = launch_split_digits_columns(Wg, g.Kg, base + p.b_planes_off, g.Og, g.Kg, false, stream);
        if (rc)
          return rc;
        rc = launch_gemm_digits(base + p.a_planes_off, base + p.b_planes_off, nullptr, col, g.M, g.Og, g.Kg, L,
                                g.Kg * L, L, stream);
      }
      if (rc)
        return rc;
      rc = launch_col2im(col, dx, g, grp, accum_x, stream);
      if (rc)
        return rc;
    }
    if (dW) {
      // digit operands of dyt^T (rows o) and col(x)^T (rows kk, gathered straight from x), contraction over the
      // pixels m
      rc = launch_split_digits_columns(dyt, g.Og, base + p.a_planes_off, g.M, g.Og, false, stream);
      if (rc)
        return rc;
      rc = launch_im2col_digits_columns(x, base + p.b_planes_off, g, grp, stream);
      if (rc)
        return rc;
      // the buffer of the unfolded gradient is free here: it takes the partial results of a split contraction
      rc = launch_gemm_digits(base + p.a_planes_off, base + p.b_planes_off, nullptr, dW + grp * g.Og * g.Kg, g.Og, g.M,
                              g.Kg, 1, g.Kg, 1, stream, accum_w, col, (size_t)g.M * g.Kg * sizeof(float));
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

size_t nbla_hip_convolution_backward_workspace_bytes(int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                                     const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                                     const int64_t *dilation, int64_t group) {
  ConvGeom g;
  if (make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group))
    return 0;
  return plan_conv_backward(g).total;
}

int nbla_hip_binary_convolution_backward_f32(const float *dy, const float *x, const float *W, const float *Wb,
                                             const float *alpha, float *dx, float *dW, float *db, int64_t outer,
                                             int64_t C, int nd, const int64_t *in_sp, int64_t O, const int64_t *kernel,
                                             const int64_t *pad, const int64_t *stride, const int64_t *dilation,
                                             int64_t group, float quantize_zero_to, int accum_x, int accum_w,
                                             int accum_b, void *workspace, size_t workspace_bytes, void *stream) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  return conv_backward(dy, x, W, Wb, alpha, dx, dW, db, g, true, quantize_zero_to, accum_x != 0, accum_w != 0,
                       accum_b != 0, workspace, workspace_bytes, stream);
}

int nbla_hip_convolution_backward_f32(const float *dy, const float *x, const float *W, float *dx, float *dW, float *db,
                                      int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                      const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                      const int64_t *dilation, int64_t group, int accum_x, int accum_w, int accum_b,
                                      void *workspace, size_t workspace_bytes, void *stream) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  return conv_backward(dy, x, W, nullptr, nullptr, dx, dW, db, g, false, 1.0f, accum_x != 0, accum_w != 0,
                       accum_b != 0, workspace, workspace_bytes, stream);
}

} // extern "C"
