// CPU oracle for nnabla's quantization function family.
//
// THIS FILE IS TEST INFRASTRUCTURE.  It restates, loop by loop and rounding by
// rounding, what nnabla's CPU ("cpu:float") implementations compute, so that the
// HIP kernels can be checked bit-for-bit (quantizers, binarized / INQ weights)
// or at tolerance (GEMM / convolution outputs).  Only tests, the smoke check and
// the CPU-baseline leg of the benchmark may load it; the product library never
// links or calls it.
//
// Every function cites the reference file:line it follows (paths relative to
// the nnabla source tree).  Arithmetic is IEEE fp32 with every operation rounded
// on its own: build with -ffp-contract=off and without -ffast-math / -march so
// that no FMA is formed (the reference's default Release build has neither
// -march nor OpenMP: CMakeLists.txt:73-74,204).
//
// Third-party arithmetic the reference delegates to Eigen 3.3.5 (not vendored
// in the reference tree: third_party/CMakeLists.txt:55):
//   * row sums (alpha = mean|W|), src/nbla/function/generic/sum.cpp:120-126
//   * GEMM, src/nbla/function/generic/affine.cpp:81-96, convolution.cpp:178-195
// The row sum below follows Eigen 3.3.5's published linear-vectorised redux
// (Core/Redux.h: two 4-lane SSE packet accumulators, combined, horizontally
// added as (l0+l2)+(l1+l3), then the scalar tail) for a 16-byte aligned row.
// The GEMM is a plain fp32 k-sequential product.  PARITY UNPINNED for the fp32
// *bits* of alpha and of GEMM/convolution outputs (only an Eigen build could pin
// their summation order); they are pinned at tolerance against float64.
// Everything else (quantizer outputs, sign-binarized weights, INQ weights and
// indicators, min/max state) is pinned bit-exactly by closed forms, invariants
// and brute force in tests/test_oracle_*.py.
//
// Known limits, same as the reference's undefined behaviour: NaN inputs to
// FixedPointQuantize (int(NaN)), bit widths >= 31.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <string>
#include <vector>

namespace {

enum { ORC_OK = 0, ORC_ERR_VALUE = 3, ORC_ERR_NOT_IMPLEMENTED = 2 };

// ---------------------------------------------------------------------------
// Helper Functions composed by the reference (each is its own pass there).
// ---------------------------------------------------------------------------

// include/nbla/function/sign.hpp:48-50
inline float sign_op(float x, float a0) {
  return (x > 0.0f) ? 1.0f : ((x < 0.0f) ? -1.0f : a0);
}

// Eigen 3.3.5 Core/Redux.h, redux_impl<Func, Derived, LinearVectorizedTraversal,
// NoUnrolling> with Packet4f (SSE2, no SSE3 hadd), as reached from
// sum.cpp:123-125 (`mx.rowwise().sum()` on a row-major map).
float eigen_row_sum(const float *row, long size) {
  const long packet = 4;
  const long aligned_size2 = (size / (2 * packet)) * (2 * packet);
  const long aligned_size = (size / packet) * packet;
  if (aligned_size == 0) {
    float res = row[0];
    for (long i = 1; i < size; ++i)
      res = res + row[i];
    return res;
  }
  float p0[4], p1[4];
  for (int l = 0; l < 4; ++l)
    p0[l] = row[l];
  if (aligned_size > packet) {
    for (int l = 0; l < 4; ++l)
      p1[l] = row[packet + l];
    for (long i = 2 * packet; i < aligned_size2; i += 2 * packet) {
      for (int l = 0; l < 4; ++l)
        p0[l] = p0[l] + row[i + l];
      for (int l = 0; l < 4; ++l)
        p1[l] = p1[l] + row[i + packet + l];
    }
    for (int l = 0; l < 4; ++l)
      p0[l] = p0[l] + p1[l];
    if (aligned_size > aligned_size2)
      for (int l = 0; l < 4; ++l)
        p0[l] = p0[l] + row[aligned_size2 + l];
  }
  // predux<Packet4f> without SSE3: tmp = a + movehl(a,a); tmp0 + tmp1
  float res = (p0[0] + p0[2]) + (p0[1] + p0[3]);
  for (long i = aligned_size; i < size; ++i)
    res = res + row[i];
  return res;
}

// y[M,N] = x[M,K] * w[K,N] (+ b[N]); affine.cpp:81-96.  fp32, k-sequential.
void sgemm_rowmajor(const float *x, const float *w, const float *b, float *y,
                    long M, long K, long N) {
  const long RB = 4;
  for (long i0 = 0; i0 < M; i0 += RB) {
    const long rb = std::min(RB, M - i0);
    for (long r = 0; r < rb; ++r)
      std::memset(y + (i0 + r) * N, 0, sizeof(float) * N);
    if (rb == RB) {
      float *y0 = y + (i0 + 0) * N, *y1 = y + (i0 + 1) * N;
      float *y2 = y + (i0 + 2) * N, *y3 = y + (i0 + 3) * N;
      for (long k = 0; k < K; ++k) {
        const float a0 = x[(i0 + 0) * K + k], a1 = x[(i0 + 1) * K + k];
        const float a2 = x[(i0 + 2) * K + k], a3 = x[(i0 + 3) * K + k];
        const float *wk = w + k * N;
        for (long j = 0; j < N; ++j) {
          const float wv = wk[j];
          y0[j] = y0[j] + a0 * wv;
          y1[j] = y1[j] + a1 * wv;
          y2[j] = y2[j] + a2 * wv;
          y3[j] = y3[j] + a3 * wv;
        }
      }
    } else {
      for (long r = 0; r < rb; ++r) {
        float *yr = y + (i0 + r) * N;
        for (long k = 0; k < K; ++k) {
          const float a = x[(i0 + r) * K + k];
          const float *wk = w + k * N;
          for (long j = 0; j < N; ++j)
            yr[j] = yr[j] + a * wk[j];
        }
      }
    }
    if (b)
      for (long r = 0; r < rb; ++r)
        for (long j = 0; j < N; ++j)
          y[(i0 + r) * N + j] = y[(i0 + r) * N + j] + b[j];
  }
}

// Convolution geometry shared by the conv entry points; convolution.cpp:41-160.
struct ConvGeom {
  int nd;
  long outer, C, O, group;
  long in_sp[3], k[3], pad[3], stride[3], dil[3], out_sp[3];
  long in_sp_size, out_sp_size, k_size, col_rows; // col_rows = (C/group)*k_size
};

int make_geom(ConvGeom &g, long outer, long C, int nd, const long *in_sp,
              long O, const long *kernel, const long *pad, const long *stride,
              const long *dil, long group) {
  if (nd < 1 || nd > 3)
    return ORC_ERR_NOT_IMPLEMENTED;
  if (group < 1 || C % group || O % group)
    return ORC_ERR_VALUE;
  g.nd = nd;
  g.outer = outer;
  g.C = C;
  g.O = O;
  g.group = group;
  g.in_sp_size = g.out_sp_size = g.k_size = 1;
  for (int i = 0; i < nd; ++i) {
    g.in_sp[i] = in_sp[i];
    g.k[i] = kernel[i];
    g.pad[i] = pad[i];
    g.stride[i] = stride[i];
    g.dil[i] = dil[i];
    const long ke = dil[i] * (kernel[i] - 1) + 1;
    g.out_sp[i] = (in_sp[i] + 2 * pad[i] - ke) / stride[i] + 1; // :97-98
    if (g.out_sp[i] <= 0 || in_sp[i] + 2 * pad[i] - ke < 0)
      return ORC_ERR_VALUE;
    g.in_sp_size *= in_sp[i];
    g.out_sp_size *= g.out_sp[i];
    g.k_size *= kernel[i];
  }
  g.col_rows = (C / group) * g.k_size;
  return ORC_OK;
}

// im2col of one sample: col[(c, kidx...), (out position...)];
// src/nbla/utils/unfold_to_patches.cpp:103-194 (zero where the tap is in the
// padding).  Rows cover all C channels (group-major, as the reference's col_).
void im2col(const ConvGeom &g, const float *xs, float *col) {
  const long rows = g.C * g.k_size;
  for (long r = 0; r < rows; ++r) {
    long rem = r;
    long kidx[3] = {0, 0, 0};
    for (int i = g.nd - 1; i >= 0; --i) {
      kidx[i] = rem % g.k[i];
      rem /= g.k[i];
    }
    const long c = rem;
    const float *xc = xs + c * g.in_sp_size;
    float *dst = col + r * g.out_sp_size;
    for (long p = 0; p < g.out_sp_size; ++p) {
      long prem = p;
      long off = 0, mul = 1;
      bool inside = true;
      for (int i = g.nd - 1; i >= 0; --i) {
        const long o = prem % g.out_sp[i];
        prem /= g.out_sp[i];
        const long pos = o * g.stride[i] + kidx[i] * g.dil[i] - g.pad[i];
        if (pos < 0 || pos >= g.in_sp[i])
          inside = false;
        off += pos * mul;
        mul *= g.in_sp[i];
      }
      dst[p] = inside ? xc[off] : 0.0f;
    }
  }
}

// convolution.cpp:161-197: per sample im2col, per group  y = W_g * col_g, bias
// added per output channel afterwards.
void conv_forward(const ConvGeom &g, const float *x, const float *w,
                  const float *b, float *y) {
  std::vector<float> col((size_t)g.C * g.k_size * g.out_sp_size);
  const long row_w = g.O / g.group;
  const long in_size = g.C * g.in_sp_size;
  const long out_size = g.O * g.out_sp_size;
  for (long n = 0; n < g.outer; ++n) {
    im2col(g, x + n * in_size, col.data());
    float *yn = y + n * out_size;
    for (long gi = 0; gi < g.group; ++gi) {
      sgemm_rowmajor(w + gi * row_w * g.col_rows,
                     col.data() + gi * g.col_rows * g.out_sp_size, nullptr,
                     yn + gi * row_w * g.out_sp_size, row_w, g.col_rows,
                     g.out_sp_size);
    }
    if (b)
      for (long o = 0; o < g.O; ++o)
        for (long p = 0; p < g.out_sp_size; ++p)
          yn[o * g.out_sp_size + p] = yn[o * g.out_sp_size + p] + b[o];
  }
}

// col2im of one sample, accumulating into dxs: fold_from_patches.cpp:22-170.
// Each column row (c, kernel index) is added into the image in row order, so an
// image element receives its taps in ascending kernel index.
void col2im_add(const ConvGeom &g, const float *col, float *dxs) {
  const long rows = g.C * g.k_size;
  for (long r = 0; r < rows; ++r) {
    long rem = r;
    long kidx[3] = {0, 0, 0};
    for (int i = g.nd - 1; i >= 0; --i) {
      kidx[i] = rem % g.k[i];
      rem /= g.k[i];
    }
    float *xc = dxs + rem * g.in_sp_size;
    const float *src = col + r * g.out_sp_size;
    for (long p = 0; p < g.out_sp_size; ++p) {
      long prem = p;
      long off = 0, mul = 1;
      bool inside = true;
      for (int i = g.nd - 1; i >= 0; --i) {
        const long o = prem % g.out_sp[i];
        prem /= g.out_sp[i];
        const long pos = o * g.stride[i] + kidx[i] * g.dil[i] - g.pad[i];
        if (pos < 0 || pos >= g.in_sp[i])
          inside = false;
        off += pos * mul;
        mul *= g.in_sp[i];
      }
      if (inside)
        xc[off] = xc[off] + src[p];
    }
  }
}

// Convolution<T>::backward_impl, convolution.cpp:199-283: the sample loop with
//   col_g = W_g^T * dy_g, folded into dx;   dW_g += dy_g * col_g(x)^T;   db += row sums of dy.
// Plain loops stand in for the Eigen products (their summation order is not restated).
void conv_backward(const ConvGeom &g, const float *dy, const float *x, const float *w, float *dx,
                   float *dw, float *db, int accum_x, int accum_w, int accum_b) {
  const long row_w = g.O / g.group, col_w = g.col_rows, L = g.out_sp_size;
  const long in_size = g.C * g.in_sp_size, out_size = g.O * L;
  std::vector<float> col((size_t)g.C * g.k_size * L);
  if (dx && !accum_x)
    std::fill(dx, dx + g.outer * in_size, 0.0f);
  if (dw && !accum_w)
    std::fill(dw, dw + g.O * col_w, 0.0f);
  if (db && !accum_b)
    std::fill(db, db + g.O, 0.0f);
  for (long n = 0; n < g.outer; ++n) {
    const float *dyn = dy + n * out_size;
    if (dx) {
      for (long gi = 0; gi < g.group; ++gi) {
        const float *wg = w + gi * row_w * col_w;
        const float *dyg = dyn + gi * row_w * L;
        float *cg = col.data() + gi * col_w * L;
        for (long j = 0; j < col_w; ++j)
          for (long p = 0; p < L; ++p) {
            float acc = 0.0f;
            for (long o = 0; o < row_w; ++o)
              acc += wg[o * col_w + j] * dyg[o * L + p];
            cg[j * L + p] = acc;
          }
      }
      col2im_add(g, col.data(), dx + n * in_size);
    }
    if (dw) {
      im2col(g, x + n * in_size, col.data());
      for (long gi = 0; gi < g.group; ++gi) {
        const float *dyg = dyn + gi * row_w * L;
        const float *cg = col.data() + gi * col_w * L;
        float *dwg = dw + gi * row_w * col_w;
        for (long o = 0; o < row_w; ++o)
          for (long j = 0; j < col_w; ++j) {
            float acc = 0.0f;
            for (long p = 0; p < L; ++p)
              acc += dyg[o * L + p] * cg[j * L + p];
            dwg[o * col_w + j] = dwg[o * col_w + j] + acc;
          }
      }
    }
    if (db)
      for (long o = 0; o < g.O; ++o) {
        float acc = 0.0f;
        for (long p = 0; p < L; ++p)
          acc += dyn[o * L + p];
        db[o] = db[o] + acc;
      }
  }
}

// Steps B and C of inq_affine.cpp:104-190 (shared verbatim by
// inq_convolution.cpp:119-205), plus step A (:95-102).
struct InqState {
  long size;
  int num_bits;
  std::vector<int> inq_iterations;
  std::string algo;
  int seed;
  long minibatch_counter;
  std::vector<float> old_weights;
  std::vector<int> old_indicators;
  std::mt19937 rgen;
  std::bernoulli_distribution rdist;
};

// Stand-in for nnabla's process-wide RandomManager generator (seed 313 by
// default, src/nbla/random_manager.cpp) used when seed == -1.
std::mt19937 &global_rgen() {
  static std::mt19937 g(313);
  return g;
}

} // namespace

extern "C" {

// ---------------------------------------------------------------------------
// FixedPointQuantize: src/nbla/function/generic/fixed_point_quantize.cpp:29-66
// ---------------------------------------------------------------------------
int orc_fixed_point_quantize(const float *x, float *y, long size, int sign,
                             int n_bits, float delta) {
  if (!(n_bits > 0 && delta > 0.))
    return ORC_ERR_VALUE; // :31-32
  const int n = sign ? n_bits - 1 : n_bits;
  if (!(n > 0))
    return ORC_ERR_VALUE; // :41-42
  const float max_ = (float)((std::pow(2, n) - 1) * delta); // :39 (float member)
  const float min_ = sign ? (float)(-max_) : 0.0f;          // :40
  for (long s = 0; s < size; ++s) {
    float y_tmp;
    if (x[s] > max_) {
      y_tmp = max_;
    } else if (x[s] < min_) {
      y_tmp = min_;
    } else {
      const bool sign_x = (x[s] < 0.0);
      const float abs_x = std::fabs(x[s]);
      // float divide, double add of 0.5, truncation, float multiply (:61)
      y_tmp = (float)(int)((abs_x / delta) + 0.5) * delta;
      y_tmp = sign_x ? -y_tmp : y_tmp;
    }
    y[s] = y_tmp;
  }
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Pow2Quantize: src/nbla/function/generic/pow2_quantize.cpp:29-82
// ---------------------------------------------------------------------------
int orc_pow2_quantize(const float *x, float *y, long size, int sign,
                      int with_zero, int n_bits, int m) {
  if (!(n_bits > 0))
    return ORC_ERR_VALUE;
  int n = sign ? n_bits - 1 : n_bits;
  n = with_zero ? n - 1 : n;
  if (!(n > 0))
    return ORC_ERR_VALUE;
  const float p_max = (float)std::pow(2., m);
  const float p_min = (float)std::pow(2., m - ((1 << n) - 1));
  const float pruning_threshold = (float)(p_min * std::pow(2., -0.5));
  for (long s = 0; s < size; ++s) {
    const float x_abs = std::fabs(x[s]);
    float q = std::pow(2.0f, std::round(std::log2(x_abs))); // powf/roundf/log2f
    if (q > p_max) {
      q = p_max;
    } else if (q < p_min && with_zero) {
      q = x_abs < pruning_threshold ? 0.0f : p_min;
    } else if (q < p_min) {
      q = p_min;
    }
    const bool sign_x = (x[s] < 0.0);
    if (sign) {
      q = sign_x ? -q : q;
    } else {
      if (with_zero)
        q = sign_x ? 0.0f : q;
      else
        q = sign_x ? p_min : q;
    }
    y[s] = q;
  }
  return ORC_OK;
}

// r = roundf(log2f(a)) as the host libm gives it: the single libm-dependent
// decision inside Pow2Quantize (pow2_quantize.cpp:60).  Exposed so tests can
// check the product's calibrated cut table against the same libm.
int orc_round_log2(float a) { return (int)std::round(std::log2(a)); }

// ---------------------------------------------------------------------------
// Min / Max reductions: src/nbla/function/generic/min.cpp:22-42, max.cpp:44-61,
// with Sum::setup_impl's "move reduced axes last" transpose (sum.cpp:44-93).
// x has shape xshape[ndim]; axes with qshape[i]==1 are reduced (keep_dims).
// ---------------------------------------------------------------------------
static void reduce_min_max(const float *x, const long *xshape, int ndim,
                           const long *qshape, float *mn, float *mx) {
  long total = 1, qsize = 1, red = 1;
  for (int i = 0; i < ndim; ++i) {
    total *= xshape[i];
    qsize *= qshape[i];
    if (qshape[i] == 1)
      red *= xshape[i];
  }
  // permutation: kept axes first (in order), reduced axes last (in order)
  std::vector<int> perm;
  for (int i = 0; i < ndim; ++i)
    if (qshape[i] != 1)
      perm.push_back(i);
  for (int i = 0; i < ndim; ++i)
    if (qshape[i] == 1)
      perm.push_back(i);
  bool identity = true;
  for (int i = 0; i < ndim; ++i)
    identity = identity && perm[i] == i;
  const float *src = x;
  std::vector<float> xt;
  if (!identity) { // transpose.cpp:91-99: materialised copy
    xt.resize(total);
    std::vector<long> xstride(ndim), tshape(ndim);
    long s = 1;
    for (int i = ndim - 1; i >= 0; --i) {
      xstride[i] = s;
      s *= xshape[i];
    }
    for (int i = 0; i < ndim; ++i)
      tshape[i] = xshape[perm[i]];
    for (long o = 0; o < total; ++o) {
      long rem = o, off = 0;
      for (int i = ndim - 1; i >= 0; --i) {
        off += (rem % tshape[i]) * xstride[perm[i]];
        rem /= tshape[i];
      }
      xt[o] = x[off];
    }
    src = xt.data();
  }
  const long outer = total / red;
  (void)qsize;
  for (long o = 0; o < outer; ++o) {
    if (mn) {
      float m = 1e+8;
      for (long i = 0; i < red; ++i) {
        const float v = src[o * red + i];
        if (v < m)
          m = v;
      }
      mn[o] = m;
    }
    if (mx) {
      float m = -1e+8;
      for (long i = 0; i < red; ++i) {
        const float v = src[o * red + i];
        if (v > m)
          m = v;
      }
      mx[o] = m;
    }
  }
}

int orc_min_max_reduce(const float *x, const long *xshape, int ndim,
                       const long *qshape, float *mn, float *mx) {
  reduce_min_max(x, xshape, ndim, qshape, mn, mx);
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// MinMaxQuantize forward: src/nbla/function/generic/min_max_quantize.cpp:130-223,
// nudge_range :353-361, nudge_qr_min_max :363-390.  qr_min / qr_max are updated
// in place (they are the function's running state); scale_out (q-shaped) is what
// the reference keeps in scale_sptr_.  Each reference pass is its own loop over
// a full-size temporary, as there.
// ---------------------------------------------------------------------------
int orc_min_max_quantize(const float *x, float *y, const long *xshape, int ndim,
                         const long *qshape, float *qr_min, float *qr_max,
                         const float *ql_min, const float *ql_max, float decay,
                         int x_min_max, int ema, float eps, float *scale_out) {
  long total = 1, qsize = 1;
  for (int i = 0; i < ndim; ++i) {
    if (qshape[i] != 1 && qshape[i] != xshape[i])
      return ORC_ERR_VALUE; // :69-81
    total *= xshape[i];
    qsize *= qshape[i];
  }
  const float decay_f = (float)decay;                    // (T)(decay_) :105
  const float one_minus = (float)(1.0 - (double)decay);  // (T)(1.0 - decay_) :106
  std::vector<float> iv(qsize);
  if (x_min_max && ema) { // :159-163, :171-175
    reduce_min_max(x, xshape, ndim, qshape, iv.data(), nullptr);
    for (long i = 0; i < qsize; ++i)
      iv[i] = iv[i] * one_minus;
    for (long i = 0; i < qsize; ++i)
      qr_min[i] = qr_min[i] * decay_f;
    for (long i = 0; i < qsize; ++i)
      qr_min[i] = qr_min[i] + iv[i];
    reduce_min_max(x, xshape, ndim, qshape, nullptr, iv.data());
    for (long i = 0; i < qsize; ++i)
      iv[i] = iv[i] * one_minus;
    for (long i = 0; i < qsize; ++i)
      qr_max[i] = qr_max[i] * decay_f;
    for (long i = 0; i < qsize; ++i)
      qr_max[i] = qr_max[i] + iv[i];
  } else if (x_min_max && !ema) { // :164-167, :176-178
    reduce_min_max(x, xshape, ndim, qshape, qr_min, nullptr);
    reduce_min_max(x, xshape, ndim, qshape, nullptr, qr_max);
  }
  // nudge_range :353-361
  for (long i = 0; i < qsize; ++i)
    if (qr_max[i] - qr_min[i] < eps)
      qr_max[i] = qr_min[i] + eps;
  // scale :188-190
  std::vector<float> scale(qsize), m_n(qsize), M_n(qsize);
  for (long i = 0; i < qsize; ++i)
    scale[i] = qr_max[i] - qr_min[i];
  for (long i = 0; i < qsize; ++i)
    iv[i] = ql_max[i] - ql_min[i];
  for (long i = 0; i < qsize; ++i)
    scale[i] = scale[i] / iv[i];
  // nudge_qr_min_max :363-390
  for (long i = 0; i < qsize; ++i) {
    const float zero_point_from_min = ql_min[i] - qr_min[i] / scale[i];
    float zero_point_nudged;
    if (zero_point_from_min <= ql_min[i])
      zero_point_nudged = ql_min[i];
    else if (zero_point_from_min >= ql_max[i])
      zero_point_nudged = ql_max[i];
    else
      zero_point_nudged = std::round(zero_point_from_min);
    m_n[i] = (ql_min[i] - zero_point_nudged) * scale[i];
    M_n[i] = (ql_max[i] - zero_point_nudged) * scale[i];
  }
  if (scale_out)
    std::memcpy(scale_out, scale.data(), sizeof(float) * qsize);
  // Broadcast (:201-209) into three full-size temporaries.
  std::vector<long> qstride(ndim);
  {
    long s = 1;
    for (int i = ndim - 1; i >= 0; --i) {
      qstride[i] = (qshape[i] == 1) ? 0 : s;
      s *= qshape[i];
    }
  }
  std::vector<float> bmin(total), bmax(total), bscale(total);
  for (long o = 0; o < total; ++o) {
    long rem = o, qi = 0;
    for (int i = ndim - 1; i >= 0; --i) {
      qi += (rem % xshape[i]) * qstride[i];
      rem /= xshape[i];
    }
    bmin[o] = m_n[qi];
    bmax[o] = M_n[qi];
    bscale[o] = scale[qi];
  }
  // :213-222, one pass per helper Function
  for (long o = 0; o < total; ++o)
    y[o] = (x[o] > bmin[o]) ? x[o] : bmin[o]; // maximum2.hpp:41
  for (long o = 0; o < total; ++o)
    y[o] = (y[o] < bmax[o]) ? y[o] : bmax[o]; // minimum2.hpp:41
  for (long o = 0; o < total; ++o)
    y[o] = y[o] - bmin[o];
  for (long o = 0; o < total; ++o)
    y[o] = y[o] / bscale[o];
  for (long o = 0; o < total; ++o)
    y[o] = std::round(y[o]); // round.hpp:42
  for (long o = 0; o < total; ++o)
    y[o] = y[o] * bscale[o];
  for (long o = 0; o < total; ++o)
    y[o] = y[o] + bmin[o];
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Affine<T>::backward_impl, affine.cpp:98-140 (plain loops in place of the Eigen
// products; their summation order is not restated), and the two binary affine
// backward passes built on it.
// ---------------------------------------------------------------------------
int orc_affine_backward(const float *dy, const float *x, const float *w, float *dx,
                        float *dw, float *db, long M, long K, long N, int accum_x,
                        int accum_w, int accum_b) {
  if (dx) { // mdx (+)= mdy * mw.transpose()
    for (long m = 0; m < M; ++m)
      for (long k = 0; k < K; ++k) {
        float acc = 0.0f;
        for (long n = 0; n < N; ++n)
          acc += dy[m * N + n] * w[k * N + n];
        dx[m * K + k] = accum_x ? dx[m * K + k] + acc : acc;
      }
  }
  if (dw) { // mdw (+)= mx.transpose() * mdy
    for (long k = 0; k < K; ++k)
      for (long n = 0; n < N; ++n) {
        float acc = 0.0f;
        for (long m = 0; m < M; ++m)
          acc += x[m * K + k] * dy[m * N + n];
        dw[k * N + n] = accum_w ? dw[k * N + n] + acc : acc;
      }
  }
  if (db) { // mdb (+)= mdy.colwise().sum()
    for (long n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (long m = 0; m < M; ++m)
        acc += dy[m * N + n];
      db[n] = accum_b ? db[n] + acc : acc;
    }
  }
  return ORC_OK;
}

// BinaryWeightAffine<T>::backward_impl, binary_weight_affine.cpp:124-146 (alpha != null) and
// BinaryConnectAffine<T>::backward_impl, binary_connect_affine.cpp:73-92 (alpha == null): Affine backward with the
// (scaled) binary weights, its weight gradient computed without accumulation and then passed through Sign's
// backward (identity, sign.hpp:48-50) onto dW.
int orc_binary_affine_backward(const float *dy, const float *x, const float *W,
                               const float *alpha, float *dx, float *dW, float *db,
                               long M, long K, long N, float quantize_zero_to,
                               int accum_x, int accum_w, int accum_b) {
  std::vector<float> ws((size_t)K * N), g;
  for (long k = 0; k < K; ++k)
    for (long n = 0; n < N; ++n) {
      const float v = W[k * N + n];
      const float b = (v > 0.0f) ? 1.0f : ((v < 0.0f) ? -1.0f : quantize_zero_to);
      ws[k * N + n] = alpha ? b * alpha[n] : b;
    }
  if (dW)
    g.resize((size_t)K * N);
  orc_affine_backward(dy, x, ws.data(), dx, dW ? g.data() : nullptr, db, M, K, N, accum_x, 0, accum_b);
  if (dW)
    for (long i = 0; i < K * N; ++i)
      dW[i] = accum_w ? dW[i] + g[i] : g[i];
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Backward passes of the three quantizers (straight-through estimators).
// ---------------------------------------------------------------------------

// FixedPointQuantize<T>::backward_impl, fixed_point_quantize.cpp:69-127.
int orc_fixed_point_quantize_backward(const float *dy, const float *x, float *dx,
                                      long size, int sign, int n_bits, float delta,
                                      int ste_fine_grained, int accum) {
  if (!(n_bits > 0 && delta > 0.))
    return ORC_ERR_VALUE;
  const int n = sign ? n_bits - 1 : n_bits;
  if (!(n > 0))
    return ORC_ERR_VALUE;
  const float max_ = (float)((std::pow(2, n) - 1) * delta);
  const float min_ = sign ? (float)(-max_) : 0.0f;
  for (long s = 0; s < size; ++s) {
    if (!ste_fine_grained) { // :69-78
      if (accum)
        dx[s] += dy[s];
      else
        dx[s] = dy[s];
    } else if (x[s] > max_) { // :84-99
      if (!accum)
        dx[s] = 0.0f;
    } else if (x[s] < min_) {
      if (!accum)
        dx[s] = 0.0f;
    } else {
      if (accum)
        dx[s] += dy[s];
      else
        dx[s] = dy[s];
    }
  }
  return ORC_OK;
}

// Pow2Quantize<T>::backward_impl, pow2_quantize.cpp:84-156.
int orc_pow2_quantize_backward(const float *dy, const float *x, float *dx, long size,
                               int sign, int with_zero, int n_bits, int m,
                               int ste_fine_grained, int accum) {
  if (!(n_bits > 0))
    return ORC_ERR_VALUE;
  int n = sign ? n_bits - 1 : n_bits;
  n = with_zero ? n - 1 : n;
  if (!(n > 0))
    return ORC_ERR_VALUE;
  const float p_max = (float)std::pow(2., m);
  for (long s = 0; s < size; ++s) {
    float c = 1.0f;
    if (ste_fine_grained) { // :97-125
      const float x_abs = std::fabs(x[s]);
      const float q = std::pow(2.0f, std::round(std::log2(x_abs)));
      if (q > p_max)
        c = 0.0f;
      if (!sign)
        c = (x[s] < 0.0) ? 0.0f : c;
      if (accum)
        dx[s] += c * dy[s];
      else
        dx[s] = c * dy[s];
    } else {
      if (accum)
        dx[s] += dy[s];
      else
        dx[s] = dy[s];
    }
  }
  return ORC_OK;
}

// MinMaxQuantize<T>::backward_impl, min_max_quantize.cpp:225-350.  qr_min / qr_max are the
// values the forward pass left, `scale` its scale_sptr_.  dx / g_qr_min / g_qr_max may be
// null (propagate_down false).  The Sum helper is a plain running sum here; the reference's
// Eigen reduction order is not restated (results are compared at tolerance).
int orc_min_max_quantize_backward(const float *dy, const float *x, float *dx,
                                  const long *xshape, int ndim, const long *qshape,
                                  const float *qr_min, const float *qr_max,
                                  const float *ql_min, const float *ql_max,
                                  const float *scale, float *g_qr_min, float *g_qr_max,
                                  int ste_fine_grained, int x_min_max, int ema,
                                  int accum_x, int accum_min, int accum_max) {
  long total = 1, qsize = 1;
  for (int i = 0; i < ndim; ++i) {
    if (qshape[i] != 1 && qshape[i] != xshape[i])
      return ORC_ERR_VALUE;
    total *= xshape[i];
    qsize *= qshape[i];
  }
  // nudge_qr_min_max :363-390 with the forward's scale
  std::vector<float> m_n(qsize), M_n(qsize);
  for (long i = 0; i < qsize; ++i) {
    const float zero_point_from_min = ql_min[i] - qr_min[i] / scale[i];
    float zero_point_nudged;
    if (zero_point_from_min <= ql_min[i])
      zero_point_nudged = ql_min[i];
    else if (zero_point_from_min >= ql_max[i])
      zero_point_nudged = ql_max[i];
    else
      zero_point_nudged = std::round(zero_point_from_min);
    m_n[i] = (ql_min[i] - zero_point_nudged) * scale[i];
    M_n[i] = (ql_max[i] - zero_point_nudged) * scale[i];
  }
  std::vector<long> qstride(ndim);
  {
    long s = 1;
    for (int i = ndim - 1; i >= 0; --i) {
      qstride[i] = (qshape[i] == 1) ? 0 : s;
      s *= qshape[i];
    }
  }
  std::vector<long> qidx(total);
  for (long o = 0; o < total; ++o) {
    long rem = o, qi = 0;
    for (int i = ndim - 1; i >= 0; --i) {
      qi += (rem % xshape[i]) * qstride[i];
      rem /= xshape[i];
    }
    qidx[o] = qi;
  }
  if (dx) { // :259-292
    for (long o = 0; o < total; ++o) {
      if (ste_fine_grained) {
        const float iv0 = (x[o] >= m_n[qidx[o]]) ? 1.0f : 0.0f; // greater_equal
        const float iv1 = (x[o] <= M_n[qidx[o]]) ? 1.0f : 0.0f; // less_equal
        float mask = iv0 * iv1;
        mask = mask * dy[o];
        dx[o] = accum_x ? mask + dx[o] : mask;
      } else {
        dx[o] = accum_x ? dy[o] + dx[o] : dy[o];
      }
    }
  }
  if (x_min_max || ema) // :294-295
    return ORC_OK;
  if (g_qr_min) { // :302-323
    std::vector<float> acc(qsize, 0.0f);
    for (long o = 0; o < total; ++o) {
      const float mask = (x[o] < m_n[qidx[o]]) ? 1.0f : 0.0f;
      acc[qidx[o]] += mask * dy[o];
    }
    for (long i = 0; i < qsize; ++i)
      g_qr_min[i] = accum_min ? g_qr_min[i] + acc[i] : acc[i];
  }
  if (g_qr_max) { // :325-348
    std::vector<float> acc(qsize, 0.0f);
    for (long o = 0; o < total; ++o) {
      const float mask = (x[o] > M_n[qidx[o]]) ? 1.0f : 0.0f;
      acc[qidx[o]] += mask * dy[o];
    }
    for (long i = 0; i < qsize; ++i)
      g_qr_max[i] = accum_max ? g_qr_max[i] + acc[i] : acc[i];
  }
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Sign: include/nbla/function/sign.hpp:48-50
// ---------------------------------------------------------------------------
void orc_sign(const float *x, float *y, long size, float alpha0) {
  for (long i = 0; i < size; ++i)
    y[i] = sign_op(x[i], alpha0);
}

// ---------------------------------------------------------------------------
// Affine: src/nbla/function/generic/affine.cpp:81-96.  b may be NULL.
// ---------------------------------------------------------------------------
int orc_affine(const float *x, const float *w, const float *b, float *y, long M,
               long K, long N) {
  sgemm_rowmajor(x, w, b, y, M, K, N);
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// BinaryWeightAffine forward: binary_weight_affine.cpp:75-122.
// W viewed [K, N]; outputs Wb [K,N], alpha [N], y [M,N].  b may be NULL.
// Passes as in the reference: Transpose -> Abs -> Sum(axis 1) -> MulScalar(1/K)
// -> Sign -> Mul2 (broadcast alpha over rows) -> Affine.
// ---------------------------------------------------------------------------
int orc_binary_weight_prepare(const float *W, float *Wb, float *alpha,
                              float *scaled, long K, long N,
                              float quantize_zero_to) {
  std::vector<float> t((size_t)K * N);
  for (long n = 0; n < N; ++n) // transpose.cpp:91-99
    for (long k = 0; k < K; ++k)
      t[n * K + k] = W[k * N + n];
  for (long i = 0; i < K * N; ++i) // abs.hpp:42
    t[i] = std::abs(t[i]);
  for (long n = 0; n < N; ++n) // sum.cpp:120-126
    alpha[n] = eigen_row_sum(t.data() + n * K, K);
  const float inv = (float)1 / K; // :68
  for (long n = 0; n < N; ++n)    // mul_scalar.hpp:43
    alpha[n] = alpha[n] * inv;
  for (long i = 0; i < K * N; ++i)
    Wb[i] = sign_op(W[i], quantize_zero_to);
  if (scaled)
    for (long k = 0; k < K; ++k) // mul2.hpp:42 with broadcast [1,N]
      for (long n = 0; n < N; ++n)
        scaled[k * N + n] = Wb[k * N + n] * alpha[n];
  return ORC_OK;
}

int orc_binary_weight_affine(const float *x, const float *W, float *Wb,
                             float *alpha, const float *b, float *y, long M,
                             long K, long N, float quantize_zero_to) {
  std::vector<float> scaled((size_t)K * N);
  orc_binary_weight_prepare(W, Wb, alpha, scaled.data(), K, N, quantize_zero_to);
  sgemm_rowmajor(x, scaled.data(), b, y, M, K, N);
  return ORC_OK;
}

// BinaryConnectAffine forward: binary_connect_affine.cpp:60-71.
int orc_binary_connect_affine(const float *x, const float *W, float *Wb,
                              const float *b, float *y, long M, long K, long N,
                              float quantize_zero_to) {
  for (long i = 0; i < K * N; ++i)
    Wb[i] = sign_op(W[i], quantize_zero_to);
  sgemm_rowmajor(x, Wb, b, y, M, K, N);
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Convolution (channel-first, N-d up to 3 spatial dims): convolution.cpp:41-197.
// x [outer, C, in_sp...], w [O, C/group, kernel...], y [outer, O, out_sp...].
// out_sp (nd longs) is written when non-NULL.  Returns the y element count via
// *y_size when non-NULL and y == NULL (shape query).
// ---------------------------------------------------------------------------
int orc_convolution(const float *x, const float *w, const float *b, float *y,
                    long outer, long C, int nd, const long *in_sp, long O,
                    const long *kernel, const long *pad, const long *stride,
                    const long *dil, long group, long *out_sp) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil,
                           group);
  if (rc)
    return rc;
  if (out_sp)
    for (int i = 0; i < nd; ++i)
      out_sp[i] = g.out_sp[i];
  if (y)
    conv_forward(g, x, w, b, y);
  return ORC_OK;
}

// BinaryWeightConvolution forward: binary_weight_convolution.cpp:73-117.
// W viewed [O, col_w]; alpha[o] = rowsum(|W[o,:]|) * ((float)1 / col_w).
int orc_binary_weight_convolution(const float *x, const float *W, float *Wb,
                                  float *alpha, const float *b, float *y,
                                  long outer, long C, int nd, const long *in_sp,
                                  long O, const long *kernel, const long *pad,
                                  const long *stride, const long *dil,
                                  long group, float quantize_zero_to) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil,
                           group);
  if (rc)
    return rc;
  const long col_w = g.col_rows;
  std::vector<float> scaled((size_t)O * col_w);
  for (long i = 0; i < O * col_w; ++i)
    scaled[i] = std::abs(W[i]);
  for (long o = 0; o < O; ++o)
    alpha[o] = eigen_row_sum(scaled.data() + o * col_w, col_w);
  const float inv = (float)1 / col_w; // :66
  for (long o = 0; o < O; ++o)
    alpha[o] = alpha[o] * inv;
  for (long i = 0; i < O * col_w; ++i)
    Wb[i] = sign_op(W[i], quantize_zero_to);
  for (long o = 0; o < O; ++o)
    for (long j = 0; j < col_w; ++j)
      scaled[o * col_w + j] = Wb[o * col_w + j] * alpha[o];
  if (y)
    conv_forward(g, x, scaled.data(), b, y);
  return ORC_OK;
}

// BinaryConnectConvolution forward: binary_connect_convolution.cpp:68-80.
int orc_binary_connect_convolution(const float *x, const float *W, float *Wb,
                                   const float *b, float *y, long outer, long C,
                                   int nd, const long *in_sp, long O,
                                   const long *kernel, const long *pad,
                                   const long *stride, const long *dil,
                                   long group, float quantize_zero_to) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil,
                           group);
  if (rc)
    return rc;
  const long wsize = O * g.col_rows;
  for (long i = 0; i < wsize; ++i)
    Wb[i] = sign_op(W[i], quantize_zero_to);
  if (y)
    conv_forward(g, x, Wb, b, y);
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// Convolution backward (also INQConvolution<T>::backward_impl, inq_convolution.cpp:220-232, which hands
// its inputs to it unchanged) and the two binary convolution backward passes.
// ---------------------------------------------------------------------------
int orc_convolution_backward(const float *dy, const float *x, const float *w, float *dx, float *dw,
                             float *db, long outer, long C, int nd, const long *in_sp, long O,
                             const long *kernel, const long *pad, const long *stride, const long *dil,
                             long group, int accum_x, int accum_w, int accum_b) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil, group);
  if (rc)
    return rc;
  conv_backward(g, dy, x, w, dx, dw, db, accum_x, accum_w, accum_b);
  return ORC_OK;
}

// BinaryWeightConvolution<T>::backward_impl, binary_weight_convolution.cpp:119-142 (alpha != null; alpha[o] scales
// output channel o) and BinaryConnectConvolution<T>::backward_impl, binary_connect_convolution.cpp:83-103
// (alpha == null): Convolution backward with the (scaled) binary weights, the weight gradient computed without
// accumulation and then passed through Sign's backward (identity) onto dW.
int orc_binary_convolution_backward(const float *dy, const float *x, const float *W, const float *alpha,
                                    float *dx, float *dW, float *db, long outer, long C, int nd,
                                    const long *in_sp, long O, const long *kernel, const long *pad,
                                    const long *stride, const long *dil, long group,
                                    float quantize_zero_to, int accum_x, int accum_w, int accum_b) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil, group);
  if (rc)
    return rc;
  const long col_w = g.col_rows;
  std::vector<float> ws((size_t)O * col_w), gw;
  for (long o = 0; o < O; ++o)
    for (long j = 0; j < col_w; ++j) {
      const float b = sign_op(W[o * col_w + j], quantize_zero_to);
      ws[o * col_w + j] = alpha ? b * alpha[o] : b;
    }
  if (dW)
    gw.resize((size_t)O * col_w);
  conv_backward(g, dy, x, ws.data(), dx, dW ? gw.data() : nullptr, db, accum_x, 0, accum_b);
  if (dW)
    for (long i = 0; i < O * col_w; ++i)
      dW[i] = accum_w ? dW[i] + gw[i] : gw[i];
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// QuantizeLinear / DequantizeLinear / Prune.
// ---------------------------------------------------------------------------
namespace {
// Offset into a broadcast parameter (sizes 1 or equal to x's) of x's flat index i.
long bcast_offset(long i, const long *xshape, const long *pshape, int ndim) {
  long off = 0, mul = 1;
  for (int d = ndim - 1; d >= 0; --d) {
    const long c = i % xshape[d];
    i /= xshape[d];
    if (pshape[d] != 1) {
      off += c * mul;
      mul *= pshape[d];
    }
  }
  return off;
}
// QuantizeLinear<T>::round, quantize_linear.cpp:78-95.
float ql_round(float v, int half_to_even) {
  if (!half_to_even)
    return std::round(v);
  const float t = std::round(v);
  if (std::abs(v - t) == 0.5)
    return (float)(std::round(v * 0.5) * 2);
  return t;
}
float ql_saturate(float v, int lo, int hi) { return v < lo ? (float)lo : (v > hi ? (float)hi : v); }
} // namespace

// QuantizeLinear<T>::forward_impl, quantize_linear.cpp:97-117 with the ranges of setup_impl :52-60; dtype 1 = BYTE,
// 2 = UBYTE.  zero_point is rounded and saturated in place, as the reference does to its input.
int orc_quantize_linear(const float *x, const float *scale, float *zero_point, float *y,
                        const long *xshape, const long *sshape, const long *zshape, int ndim,
                        int half_to_even, int narrow_range, int dtype) {
  int lo, hi;
  if (dtype == 1) {
    lo = narrow_range ? -127 : -128, hi = 127;
  } else if (dtype == 2) {
    lo = narrow_range ? 1 : 0, hi = 255;
  } else {
    return ORC_ERR_VALUE;
  }
  long size = 1, zsize = 1;
  for (int d = 0; d < ndim; ++d) {
    if ((sshape[d] != 1 && sshape[d] != xshape[d]) || (zshape[d] != 1 && zshape[d] != xshape[d]))
      return ORC_ERR_VALUE;
    size *= xshape[d];
    zsize *= zshape[d];
  }
  for (long i = 0; i < size; ++i)
    y[i] = x[i] / scale[bcast_offset(i, xshape, sshape, ndim)]; // Div2
  for (long i = 0; i < size; ++i)
    y[i] = ql_round(y[i], half_to_even);
  for (long i = 0; i < zsize; ++i)
    zero_point[i] = ql_saturate(ql_round(zero_point[i], half_to_even), lo, hi);
  for (long i = 0; i < size; ++i)
    y[i] = y[i] + zero_point[bcast_offset(i, xshape, zshape, ndim)]; // Add2
  for (long i = 0; i < size; ++i)
    y[i] = ql_saturate(y[i], lo, hi);
  return ORC_OK;
}

// DequantizeLinear<T>::forward_impl, dequantize_linear.cpp:55-67: Sub2 then Mul2.
int orc_dequantize_linear(const float *x, const float *scale, const float *zero_point, float *y,
                          const long *xshape, const long *sshape, const long *zshape, int ndim) {
  long size = 1;
  for (int d = 0; d < ndim; ++d) {
    if ((sshape[d] != 1 && sshape[d] != xshape[d]) || (zshape[d] != 1 && zshape[d] != xshape[d]))
      return ORC_ERR_VALUE;
    size *= xshape[d];
  }
  for (long i = 0; i < size; ++i)
    y[i] = x[i] - zero_point[bcast_offset(i, xshape, zshape, ndim)];
  for (long i = 0; i < size; ++i)
    y[i] = y[i] * scale[bcast_offset(i, xshape, sshape, ndim)];
  return ORC_OK;
}

// x branch of the two backward passes (quantize_linear.cpp:137-147: dy / scale; dequantize_linear.cpp:88-98:
// dy * scale), added to dx when accum.
int orc_linear_quantize_backward(const float *dy, const float *scale, float *dx, const long *xshape,
                                 const long *sshape, int ndim, int dequantize, int accum) {
  long size = 1;
  for (int d = 0; d < ndim; ++d)
    size *= xshape[d];
  for (long i = 0; i < size; ++i) {
    const float s = scale[bcast_offset(i, xshape, sshape, ndim)];
    const float g = dequantize ? dy[i] * s : dy[i] / s;
    dx[i] = accum ? dx[i] + g : g;
  }
  return ORC_OK;
}

// Prune<T>::setup_impl / forward_impl, prune.cpp:27-70.
int orc_prune(const float *x, float *y, long size, float rate) {
  if (!(rate >= 0 && rate <= 1))
    return ORC_ERR_VALUE;
  if (size == 0)
    return ORC_OK;
  const int x_size = (int)size;
  const int thresh_idx = (int)((x_size - 1) * rate);
  std::vector<float> buffer(x, x + size);
  std::sort(buffer.begin(), buffer.end(), [](float i, float j) { return std::abs(i) < std::abs(j); });
  float thresh_val = std::abs(buffer[thresh_idx]);
  thresh_val += rate == 1.0 ? 1.0 : 0.0;
  for (long s = 0; s < size; ++s)
    y[s] = (std::abs(x[s]) < thresh_val) ? 0.0f : x[s];
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// INQ (INQAffine / INQConvolution share the weight logic).
//   inq_affine.cpp:34-79 (setup), :82-205 (forward), inq_convolution.cpp:35-238.
// ---------------------------------------------------------------------------
void *orc_inq_create(long size, int num_bits, const int *inq_iterations,
                     int n_iterations, const char *selection_algorithm,
                     int seed) {
  std::string algo(selection_algorithm);
  if (algo != "largest_abs" && algo != "random")
    return nullptr; // :53-58
  InqState *s = new InqState();
  s->size = size;
  s->num_bits = num_bits;
  s->inq_iterations.assign(inq_iterations, inq_iterations + n_iterations);
  s->algo = algo;
  s->seed = seed;
  s->minibatch_counter = 0;
  s->old_weights.assign(size, 0.0f);
  s->old_indicators.assign(size, 0);
  if (algo == "random") { // :70-74 (seed -1 draws from the global generator)
    s->rgen = std::mt19937(seed == -1 ? 313u : (unsigned)seed);
    s->rdist = std::bernoulli_distribution(0.5);
  }
  return s;
}

void orc_inq_destroy(void *h) { delete static_cast<InqState *>(h); }

long orc_inq_counter(void *h) {
  return static_cast<InqState *>(h)->minibatch_counter;
}

// Steps A, B, C of the forward (:95-190): rewrites weights and indicators in
// place.  n1_out / n2_out receive the exponent range when non-NULL.
int orc_inq_quantize_weights(void *h, float *weights, int *indicators,
                             int *n1_out, int *n2_out) {
  InqState *s = static_cast<InqState *>(h);
  const long size = s->size;
  std::mt19937 &rgen = s->seed == -1 ? global_rgen() : s->rgen;
  // A
  for (long i = 0; i < size; ++i)
    if (s->old_indicators[i] == 1)
      weights[i] = s->old_weights[i];
  // B
  if (std::find(s->inq_iterations.begin(), s->inq_iterations.end(),
                (int)s->minibatch_counter) != s->inq_iterations.end()) {
    if (s->inq_iterations.back() == (int)s->minibatch_counter) {
      for (long i = 0; i < size; ++i)
        indicators[i] = 1;
    } else if (s->algo == "largest_abs") {
      std::vector<size_t> indices(size);
      std::iota(indices.begin(), indices.end(), 0);
      std::sort(indices.begin(), indices.end(), [&](size_t a, size_t b) {
        return std::abs(weights[a]) > std::abs(weights[b]);
      });
      int num_learnable = 0;
      for (long i = 0; i < size; ++i)
        if (indicators[i] == 0)
          num_learnable++;
      int num_fixed = 0;
      for (long i = 0; i < size; ++i) {
        if (indicators[indices[i]] == 0) {
          indicators[indices[i]] = 1;
          num_fixed++;
        }
        if (num_fixed >= num_learnable / 2)
          break;
      }
    } else {
      for (long i = 0; i < size; ++i)
        if (indicators[i] == 0)
          indicators[i] = s->rdist(rgen);
    }
  }
  // C
  float max_absval = 0.0f;
  for (long i = 0; i < size; ++i)
    if (std::abs(weights[i]) > max_absval)
      max_absval = std::abs(weights[i]);
  if (max_absval == 0.0f)
    max_absval = 1.0f;
  const int n1 =
      (int)(std::floor(std::log2(max_absval)) +
            (std::log2(max_absval) - std::floor(std::log2(max_absval)) >=
             std::log2(1.5)));
  const int n2 = n1 + 1 - (int)std::pow(2, s->num_bits - 2);
  const float pruning_threshold = std::pow(2, n2 - 1);
  for (long i = 0; i < size; ++i) {
    if (indicators[i] == 1) {
      if (std::abs(weights[i]) < pruning_threshold) {
        weights[i] = 0.0f;
      } else {
        const float sg = (weights[i] < 0.0) ? -1.0 : 1.0;
        const float b = std::log2(std::abs(weights[i]));
        const float d = 0.58496250072115619;
        int e = (int)(std::floor(b) + (b - std::floor(b) >= d));
        if (e > n1)
          e = n1;
        if (e < n2)
          e = n2;
        weights[i] = std::ldexp(sg, e);
      }
    }
  }
  if (n1_out)
    *n1_out = n1;
  if (n2_out)
    *n2_out = n2;
  return ORC_OK;
}

// Steps E, F (:199-204): bump the counter, snapshot weights and indicators.
int orc_inq_commit(void *h, const float *weights, const int *indicators) {
  InqState *s = static_cast<InqState *>(h);
  s->minibatch_counter++;
  std::memcpy(s->old_weights.data(), weights, sizeof(float) * s->size);
  std::memcpy(s->old_indicators.data(), indicators, sizeof(int) * s->size);
  return ORC_OK;
}

// A stand-alone Bernoulli(0.5) stream identical to the one INQ's "random" selection consumes
// (std::mt19937 + std::bernoulli_distribution, inq_affine.cpp:70-74,147): lets a test feed the same draws to
// an implementation that takes them through a callback.
void *orc_bernoulli_create(int seed) {
  InqState *s = new InqState();
  s->rgen = std::mt19937((unsigned)seed);
  s->rdist = std::bernoulli_distribution(0.5);
  return s;
}
void orc_bernoulli_draw(void *h, unsigned char *out, long count) {
  InqState *s = static_cast<InqState *>(h);
  for (long i = 0; i < count; ++i)
    out[i] = s->rdist(s->rgen) ? 1 : 0;
}

// The two libm-dependent decisions of step C, exposed for table checks:
// e(a) = floor(log2f(a)) + (frac >= (float)log2(1.5)) for a weight (:176-179)
int orc_inq_exponent(float a) {
  const float b = std::log2(a);
  const float d = 0.58496250072115619;
  return (int)(std::floor(b) + (b - std::floor(b) >= d));
}
// n1(max) with the *double* comparison of :161-164
int orc_inq_n1(float max_absval) {
  return (int)(std::floor(std::log2(max_absval)) +
               (std::log2(max_absval) - std::floor(std::log2(max_absval)) >=
                std::log2(1.5)));
}

// INQAffine forward (:82-205): W [K,N] and indicators are rewritten in place.
int orc_inq_affine(void *h, const float *x, float *W, int *indicators,
                   const float *b, float *y, long M, long K, long N) {
  orc_inq_quantize_weights(h, W, indicators, nullptr, nullptr);
  sgemm_rowmajor(x, W, b, y, M, K, N);
  return orc_inq_commit(h, W, indicators);
}

// INQConvolution forward: inq_convolution.cpp:104-238.
int orc_inq_convolution(void *h, const float *x, float *W, int *indicators,
                        const float *b, float *y, long outer, long C, int nd,
                        const long *in_sp, long O, const long *kernel,
                        const long *pad, const long *stride, const long *dil,
                        long group) {
  ConvGeom g;
  const int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dil,
                           group);
  if (rc)
    return rc;
  orc_inq_quantize_weights(h, W, indicators, nullptr, nullptr);
  conv_forward(g, x, W, b, y);
  return orc_inq_commit(h, W, indicators);
}

} // extern "C"
