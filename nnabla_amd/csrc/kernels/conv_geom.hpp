// Convolution geometry shared by the convolution entry points.
#pragma once
#include "common.hpp"

namespace nbla_hip {

constexpr int kMaxSpatial = 3;

// Geometry normalised to three spatial dimensions (leading ones of size 1).
struct ConvGeom {
  int64_t outer, C, O, group;
  int in_sp[kMaxSpatial], k[kMaxSpatial], pad[kMaxSpatial], stride[kMaxSpatial], dil[kMaxSpatial],
      out_sp[kMaxSpatial];
  int64_t in_sp_size, out_sp_size, k_size;
  int64_t Cg, Og, Kg; // per group: input channels, output channels, contraction length
  int64_t M;          // outer * out_sp_size
};

// Value of the unfolded matrix at (pixel m, column k) for group `grp`
// (unfold_to_patches.cpp:103-194: zero where the tap falls into the padding).
__device__ __forceinline__ float col_value(const float *__restrict__ x, const ConvGeom &g, int64_t grp, int64_t m,
                                           int64_t k) {
  const int64_t n = m / g.out_sp_size;
  int64_t p = m - n * g.out_sp_size;
  const int o2 = (int)(p % g.out_sp[2]);
  p /= g.out_sp[2];
  const int o1 = (int)(p % g.out_sp[1]);
  const int o0 = (int)(p / g.out_sp[1]);
  int64_t t = k;
  const int k2 = (int)(t % g.k[2]);
  t /= g.k[2];
  const int k1 = (int)(t % g.k[1]);
  t /= g.k[1];
  const int k0 = (int)(t % g.k[0]);
  const int64_t c = grp * g.Cg + t / g.k[0];
  const int i0 = o0 * g.stride[0] + k0 * g.dil[0] - g.pad[0];
  const int i1 = o1 * g.stride[1] + k1 * g.dil[1] - g.pad[1];
  const int i2 = o2 * g.stride[2] + k2 * g.dil[2] - g.pad[2];
  if ((unsigned)i0 >= (unsigned)g.in_sp[0] || (unsigned)i1 >= (unsigned)g.in_sp[1] ||
      (unsigned)i2 >= (unsigned)g.in_sp[2])
    return 0.0f;
  return x[(n * g.C + c) * g.in_sp_size + ((int64_t)i0 * g.in_sp[1] + i1) * g.in_sp[2] + i2];
}

// Validates and normalises the arguments (the checks of Convolution<T>::setup_impl, convolution.cpp:41-160).
int make_geom(ConvGeom &g, int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O, const int64_t *kernel,
              const int64_t *pad, const int64_t *stride, const int64_t *dil, int64_t group);

// Unfolded activations of group `grp`, as the int8 digit MFMA operand [M, Kg] or as plain fp32 [M, Kg].
int launch_im2col_digits(const float *x, void *xdigits, void *scratch, const ConvGeom &g, int64_t grp,
                         hipStream_t stream);
// (run_if, device memory, may be null: the launch does nothing unless the word it points to is non-zero)
int launch_im2col_f32(const float *x, float *col, const ConvGeom &g, int64_t grp, hipStream_t stream,
                      const int *run_if = nullptr);
// col(x)^T (rows = unfolded columns, contraction over the output positions) as a digit operand with one scale per
// input channel.
int launch_im2col_digits_columns(const float *x, void *digits, const ConvGeom &g, int64_t grp, hipStream_t stream);

} // namespace nbla_hip
