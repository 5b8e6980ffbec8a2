// Pieces shared by the forward and backward quantizer kernels.
#pragma once
#include "common.hpp"

namespace nbla_hip {

typedef float float4_t __attribute__((ext_vector_type(4)));

// (x shape, q shape) collapsed to element index = (r0 * K + k) * R1 + r1 with k
// the kept (per-channel) index and r0, r1 the reduced ones.
struct MinMaxLayout {
  int64_t R0, K, R1, total;
  bool ok;
};

// Any pattern of kept and reduced axes, for the strided kernels: the kept axes (row-major, as the q tensors are laid
// out) and the reduced axes (row-major: the order in which Sum / Min / Max scan a slice once the reduced axes have
// been moved to the back, sum.cpp:44-75) with their element strides in x.
struct MinMaxAxes {
  int nkept, nred;
  int64_t ksize[8], kstride[8], rsize[8], rstride[8];
};
inline bool split_axes(const int64_t *xshape, int ndim, const int64_t *qshape, MinMaxAxes &A) {
  A.nkept = A.nred = 0;
  int64_t stride = 1;
  int64_t strides[32];
  if (ndim > 32)
    return false;
  for (int i = ndim - 1; i >= 0; --i) {
    strides[i] = stride;
    stride *= xshape[i];
  }
  for (int i = 0; i < ndim; ++i) {
    if (xshape[i] == 1)
      continue;
    if (qshape[i] != 1) {
      if (A.nkept == 8)
        return false;
      A.ksize[A.nkept] = xshape[i], A.kstride[A.nkept++] = strides[i];
    } else {
      if (A.nred == 8)
        return false;
      A.rsize[A.nred] = xshape[i], A.rstride[A.nred++] = strides[i];
    }
  }
  return true;
}

inline MinMaxLayout collapse(const int64_t *xshape, int ndim, const int64_t *qshape) {
  // runs of (kept?) axes, ignoring size-1 axes
  int64_t sizes[3] = {1, 1, 1};
  int stage = 0; // 0: leading reduced, 1: kept, 2: trailing reduced
  MinMaxLayout L{1, 1, 1, 1, true};
  for (int i = 0; i < ndim; ++i) {
    const int64_t s = xshape[i];
    L.total *= s;
    if (s == 1)
      continue;
    const bool kept = qshape[i] != 1;
    if (kept) {
      if (stage == 0)
        stage = 1;
      else if (stage == 2)
        L.ok = false; // kept, reduced, kept: not a single (R0, K, R1) pattern
      sizes[1] *= s;
    } else {
      if (stage == 1)
        stage = 2;
      sizes[stage == 0 ? 0 : 2] *= s;
    }
  }
  L.R0 = sizes[0];
  L.K = sizes[1];
  L.R1 = sizes[2];
  if (!L.ok) { // general pattern (strided kernels): K kept indices, each with R1 reduced elements
    L.R1 = L.R0 * L.R1;
    L.R0 = 1;
  }
  if (L.K == 1) { // per-tensor: one flat run
    L.R1 = L.R0 * L.R1;
    L.R0 = 1;
  }
  return L;
}


// nudge_qr_min_max (min_max_quantize.cpp:363-390): the representable range [m', M'] whose zero point is an integer
// level, one rounded fp32 operation at a time.
__host__ __device__ inline void nudge_qr_min_max(float qr_min, float ql_min, float ql_max, float scale, float &m_n,
                                                  float &M_n) {
  const float zp_from_min = ql_min - qr_min / scale;
  float zp;
  if (zp_from_min <= ql_min)
    zp = ql_min;
  else if (zp_from_min >= ql_max)
    zp = ql_max;
  else {
    const float r = truncf(zp_from_min); // std::round: halves away from zero
    const float d = fabsf(zp_from_min - r);
    zp = (d >= 0.5f) ? r + copysignf(1.0f, zp_from_min) : r;
  }
  m_n = (ql_min - zp) * scale;
  M_n = (ql_max - zp) * scale;
}

} // namespace nbla_hip
