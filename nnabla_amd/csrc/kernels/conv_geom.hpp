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
