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


// Offset in x of index idx over the axes (size, stride), row-major.
__device__ __forceinline__ int64_t strided_offset(int64_t idx, int n, const int64_t *size, const int64_t *stride) {
  int64_t off = 0;
  for (int d = n - 1; d >= 0; --d) {
    const int64_t q = idx / size[d];
    off += (idx - q * size[d]) * stride[d];
    idx = q;
  }
  return off;
}

// A pattern whose kept axes are separated by reduced ones and whose innermost axis is kept (q shape (C, 1, W)): the
// kept index is (ko, w) with w along the contiguous axis, the reduced index (ro, ri) with ri along the innermost
// reduced axis.  The kernels of this form put the lanes along w, so every line of x is read once, and walk the
// reduced index in row-major order like the reference's scan.
struct MinMaxInner {
  bool ok;
  int64_t Ko, Wk;        // kept: outer combinations, innermost (contiguous) extent
  int64_t Rout, Rin;     // reduced: outer combinations, innermost extent
  int64_t rin_stride;    // element stride of the innermost reduced axis
  int tw;                // lanes along w: the power of two covering min(Wk, 64)
};
inline MinMaxInner inner_form(const MinMaxAxes &A) {
  MinMaxInner I;
  I.ok = A.nkept >= 1 && A.nred >= 1 && A.kstride[A.nkept - 1] == 1;
  if (!I.ok)
    return I;
  I.Wk = A.ksize[A.nkept - 1];
  I.Ko = 1;
  for (int d = 0; d + 1 < A.nkept; ++d)
    I.Ko *= A.ksize[d];
  I.Rin = A.rsize[A.nred - 1];
  I.rin_stride = A.rstride[A.nred - 1];
  I.Rout = 1;
  for (int d = 0; d + 1 < A.nred; ++d)
    I.Rout *= A.rsize[d];
  I.tw = 1;
  while (I.tw < 64 && I.tw < I.Wk)
    I.tw *= 2;
  I.ok = I.Ko < ((int64_t)1 << 31);
  return I;
}

// Blocks per kept outer index of the kernels of this form: about 2048 blocks in all, each a run of outer reduced
// indices.
inline int64_t inner_chunks(const MinMaxInner &I) {
  int64_t want = (2048 + I.Ko - 1) / I.Ko;
  if (want > I.Rout)
    want = I.Rout;
  const int64_t cap = I.Ko >= 32 ? 64 : 1024;
  if (want > cap)
    want = cap;
  return want < 1 ? 1 : want;
}
// Every kept axis behind every reduced one (ranges per column of a matrix, q shape (1, 1, W)): runs of one element,
// which the kernels that walk runs of R1 elements would visit one block at a time; the kernels with the lanes along
// the kept axis take such a layout.
inline bool trailing_kept(const MinMaxLayout &L) { return L.ok && L.R1 == 1 && L.K > 1 && L.R0 > 1; }

// The inner-kept form (MinMaxInner).  Block (ko, chunk): the outer reduced indices ro = chunk, chunk + nchunks, ... are
// not what it takes -- it takes the contiguous run [chunk * per, (chunk + 1) * per) so that its first-zero index grows
// along its scan.  Lane = (row slot, w): the block's 256 threads cover 256 / tw rows of tw columns per step; columns
// beyond 64 are walked in further passes over the block's rows.
struct InnerWalk {
  const float *base;   // x at (ko, w = 0)
  int64_t ro_begin, ro_end;
};
__device__ __forceinline__ InnerWalk inner_walk(const float *x, const MinMaxAxes &A, const MinMaxInner &I, int64_t ko,
                                                int chunk, int nchunks) {
  InnerWalk w;
  w.base = x + (A.nkept > 1 ? strided_offset(ko, A.nkept - 1, A.ksize, A.kstride) : 0);
  const int64_t per = (I.Rout + nchunks - 1) / nchunks;
  w.ro_begin = (int64_t)chunk * per;
  w.ro_end = w.ro_begin + per < I.Rout ? w.ro_begin + per : I.Rout;
  return w;
}
// kVec = 4: Wk a multiple of four and x (y) 16-byte aligned: a lane owns four consecutive columns (one 128-bit
// access per row) and the plan's tw counts such quads.
template <int kVec> struct InnerRow;
template <> struct InnerRow<1> {
  float v[1];
  __device__ __forceinline__ void load(const float *p) { v[0] = *p; }
  __device__ __forceinline__ void fill(float f) { v[0] = f; }
};
template <> struct InnerRow<4> {
  float v[4];
  __device__ __forceinline__ void load(const float *p) {
    const float4_t q = *reinterpret_cast<const float4_t *>(p);
    v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
  }
  __device__ __forceinline__ void fill(float f) { v[0] = v[1] = v[2] = v[3] = f; }
};

// The counterpart for patterns whose innermost axis is reduced (q shape (C, H, 1), or (1, C, 1, 1) over short
// rows): a run of Rin contiguous elements belongs to one range.  T lanes share a run (each kVec consecutive
// elements per step), 256 / T runs of consecutive kept indices are in flight per step, and a block (tile of kept
// indices, chunk) walks a run of the outer reduced indices in row-major order like the reference's scan.
struct MinMaxRows {
  bool ok;
  int64_t K, Rin, Rout; // kept indices, extent of the innermost reduced axis, combinations of the other reduced axes
};
inline MinMaxRows row_form(const MinMaxAxes &A) {
  MinMaxRows R;
  R.ok = A.nkept >= 1 && A.nred >= 1 && A.rstride[A.nred - 1] == 1;
  if (!R.ok)
    return R;
  R.K = 1;
  for (int d = 0; d < A.nkept; ++d)
    R.K *= A.ksize[d];
  R.Rin = A.rsize[A.nred - 1];
  R.Rout = 1;
  for (int d = 0; d + 1 < A.nred; ++d)
    R.Rout *= A.rsize[d];
  R.ok = R.K < ((int64_t)1 << 31) && R.Rin < ((int64_t)1 << 31);
  return R;
}
// lanes per run for kVec elements per lane and step: the power of two covering the run, at most 64
inline int row_lanes(const MinMaxRows &R, int vec) {
  int t = 1;
  while (t < 64 && (int64_t)t * vec < R.Rin)
    t *= 2;
  return t;
}
// Blocks per tile of kept indices (independent of the lanes per run, which the pointers' alignment decides).
inline int64_t row_chunks(const MinMaxRows &R) {
  const int64_t tiles = (R.K + 3) / 4;
  int64_t want = (4096 + tiles - 1) / tiles;
  if (want > R.Rout)
    want = R.Rout;
  if (want > 1024)
    want = 1024;
  return want < 1 ? 1 : want;
}
// Short runs per channel (q shape (1, C, 1, 1) over rows of fewer than 256 elements) take this form as well.
inline bool short_rows(const MinMaxLayout &L) { return L.ok && L.K > 1 && L.R1 > 1 && L.R1 < 256; }
struct RowWalk {
  int64_t ro_begin, ro_end;
};
__device__ __forceinline__ RowWalk row_walk(const MinMaxRows &R, int chunk, int nchunks) {
  RowWalk w;
  const int64_t per = (R.Rout + nchunks - 1) / nchunks;
  w.ro_begin = (int64_t)chunk * per;
  w.ro_end = w.ro_begin + per < R.Rout ? w.ro_begin + per : R.Rout;
  return w;
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
