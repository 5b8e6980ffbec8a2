// Entry points shared between the translation units of the kernel library (not part of the C-ABI).
#pragma once
#include "common.hpp"

namespace nbla_hip {

// fp32 MFMA product y = (x . w) * colscale + bias; w is [K, N], or [N, K] when trans_b.  Output element (m, n) is
// written at y[(m / inner) * outer_stride + n * n_stride + (m % inner)].
// `run_if` (device memory, may be null): the launch does nothing unless the word it points to is non-zero when the
// kernel starts -- the fallback of a product whose operand turned out not to be expressible in its fast form, decided
// on the device so that the host never waits for the answer.
// `kscale` (may be null) scales x along the contraction (x[m, k] * kscale[k]); `accumulate` adds to y.
int launch_gemm_f32_mapped(const float *x, const float *w, bool trans_b, const float *colscale, const float *bias,
                           float *y, int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride,
                           int64_t n_stride, hipStream_t stream, const int *run_if = nullptr,
                           const float *kscale = nullptr, bool accumulate = false);
int launch_gemm_f32(const float *x, const float *w, const float *colscale, const float *bias, float *y, int64_t M,
                    int64_t K, int64_t N, hipStream_t stream, const int *run_if = nullptr);
// Sets `count` 32-bit words to zero with a kernel (a memset node must not be recorded into a captured graph).
int launch_clear_words(void *dst, size_t count, hipStream_t stream);

// Bit-weight product with the choice of store orientation: swap_out makes consecutive lanes write consecutive m
// (for outputs whose m index is the contiguous one, e.g. convolution results [batch, O, Ho*Wo]).  keep_bad_rows: rows
// of the digit operand marked as holding a non-finite value are left as they are in y instead of being set to NaN.
// skip_if (device memory, may be null): the launches do nothing when the word it points to is non-zero as they start
// (the packed bits turned out not to express the weights; the caller's fp32 product runs instead).
int launch_gemm_bits(const void *xsplit, const uint32_t *bits, const float *alpha, const float *bias, float *y,
                     int64_t M, int64_t K, int64_t N, int64_t inner, int64_t outer_stride, int64_t n_stride,
                     bool swap_out, hipStream_t stream, bool accumulate = false, void *split_ws = nullptr,
                     size_t split_ws_bytes = 0, bool keep_bad_rows = false, const int *skip_if = nullptr);
// The same product for a convolution with the unfold fused in: the rows are the unfolded windows of x (group `grp`),
// converted to digits inside the kernel; y is [sample, O, output position].  gemm_bits_unfold_applies tells whether
// the geometry is covered (otherwise: launch_im2col_digits + launch_gemm_bits).  row_shift (may be null): M words that
// receive the rows' scale exponents, kBadRow for a window holding a NaN or an infinity (all its outputs are NaN).
struct ConvGeom;
bool gemm_bits_unfold_applies(const ConvGeom &g);
int launch_gemm_bits_unfold(const float *x, const ConvGeom &g, int64_t grp, const uint32_t *bits, const float *alpha,
                            const float *bias, float *y, hipStream_t stream, int32_t *row_shift = nullptr);
// y = x . W (+ bias) for at most 16 rows of x and real-valued weights [K, N]: one fp32 pass over W
// (affine_few_rows.hip).  The workspace holds the partial results of the slabs of K.
bool affine_few_rows_applies(const float *x, const float *W, const float *y, int64_t M, int64_t K, int64_t N);
size_t affine_few_rows_workspace_bytes(int64_t M, int64_t K, int64_t N);
int launch_affine_few_rows(const float *x, const float *W, const float *bias, float *y, int64_t M, int64_t K, int64_t N,
                           void *workspace, size_t workspace_bytes, hipStream_t stream);
// Grouped convolutions whose groups are too small for the matrix cores (depthwise, ResNeXt-style), all groups in one
// launch, plain fp32 (conv_direct.hip).  w: the weights [O, Kg] (for a binary convolution the materialised signs),
// scale (may be null): alpha[o].  launch_conv_direct_binarize writes Wb = Sign(W) and alpha (may be null) for all
// channels.  Backward: w as in the forward, or with take_sign the real-valued weights whose signs were used.
bool conv_direct_applies(const ConvGeom &g);
bool conv_direct_forward_applies(const ConvGeom &g); // (also a single group of very few input channels, many taps)
// The weight gradient of few weights under many windows in fp32 (all groups); scratch: M * Kg floats are enough.
bool conv_direct_dw_applies(const ConvGeom &g);
int launch_conv_direct_dw(const float *dy, const float *x, float *dW, const ConvGeom &g, bool accum, void *scratch,
                          size_t scratch_bytes, hipStream_t stream);
int launch_conv_direct_binarize(const float *W, float *Wb, float *alpha, const ConvGeom &g, float zero_to,
                                hipStream_t stream);
int launch_conv_direct_forward(const float *x, const float *w, const float *scale, const float *bias, float *y,
                               const ConvGeom &g, hipStream_t stream);
bool conv_direct_dx_applies(const ConvGeom &g);
int launch_conv_direct_dx(const float *dy, const float *w, const float *scale, float *dx, const ConvGeom &g, bool accum,
                          bool take_sign, float zero_to, float *scratch, size_t scratch_bytes, hipStream_t stream);
int launch_conv_direct_db(const float *dy, float *db, const ConvGeom &g, bool accum, float *scratch,
                          size_t scratch_bytes, hipStream_t stream);
int launch_conv_direct_backward(const float *dy, const float *x, const float *w, const float *scale, float *dx,
                                float *dW, float *db, const ConvGeom &g, bool accum_x, bool accum_w, bool accum_b,
                                bool take_sign, float zero_to, float *scratch, size_t scratch_bytes,
                                hipStream_t stream);
// The binary convolution forward with the unfold done by LDS addressing (conv_slab.hip), two launches per group:
// launch_conv_slab_prepare reads the group's weights [Og, Cg, taps] once and writes Wb = Sign(W) (may be null) and,
// into `prepared` (conv_slab_prepared_bytes, 16-byte aligned), the packed bits in (tap, channel) order with the
// partial |W| sums and zero counts; launch_conv_slab multiplies, forming alpha = mean |W| from the partial sums when
// alpha_out is not null (and writing it there), and writes the number of weights that are neither negative nor
// positive to *zero_count when that is not null.  alpha_out and bias belong to the group; y is the whole output.
bool conv_slab_applies(const ConvGeom &g);
size_t conv_slab_prepared_bytes(const ConvGeom &g);
// The plan's figures for a geometry it covers: windows per block, blocks per sample, the input positions its LDS
// holds per block, LDS bytes.  Host only.
bool conv_slab_plan_summary(const ConvGeom &g, int32_t out[4]);
int launch_conv_slab_prepare(const float *Wg, float *Wbg, void *prepared, const ConvGeom &g, float zero_to,
                             hipStream_t stream);
// in_scale (may be null): input channel c of the group is multiplied by in_scale[c] before anything else; accumulate:
// y += instead of y =.  redo_w (may be null; ignored with in_scale or accumulate): the group's Sign(W) [Og, Cg * taps],
// from which the outputs of a window holding a NaN or an infinity are recomputed one by one as the reference's product
// gives them; without it all outputs of such a window are NaN.
int launch_conv_slab(const float *x, const ConvGeom &g, int64_t grp, const void *prepared, float *alpha_out,
                     int *zero_count, const float *bias, float *y, hipStream_t stream, const float *in_scale = nullptr,
                     bool accumulate = false, const float *redo_w = nullptr);
// The same product as the input gradient of a binary convolution of unit stride: conv_slab_transposed_geom gives the
// geometry of the convolution dx = conv(dy * alpha, flipped Sign(W)^T) (false when the product does not cover it),
// launch_conv_slab_prepare_transposed writes its packed bits from the group's weights [Og, Cg, taps]
// (conv_slab_prepared_bytes of the transposed geometry), launch_conv_slab runs it with dy as x and alpha as in_scale.
bool conv_slab_transposed_geom(const ConvGeom &g, ConvGeom &t);
int launch_conv_slab_prepare_transposed(const float *Wg, void *prepared, const ConvGeom &g, float zero_to,
                                        hipStream_t stream);
// Digit operand of the rows of x (nbla_hip_split_digits_scaled_f32) for a caller that holds materialised weights
// Wb [K, N] (* alpha[n], + bias[n]): rows holding a NaN or an infinity get their outputs y[m, :] computed by the
// splitting kernel itself, as fp32 dot products in the reference's order.  *redone tells whether that happened (only
// the one-pass kernel for rows of up to 16384 values does it, and only without a column scale); the product is then
// launched with keep_bad_rows, otherwise the caller recomputes those rows after the product.
struct RowRedo {
  const float *Wb, *alpha, *bias;
  float *y;
  int64_t N;
};
int launch_split_digits_rows_redo(const float *x, int64_t ldx, const float *colscale, void *xdigits, int64_t M,
                                  int64_t K, const RowRedo *redo, bool *redone, hipStream_t stream);
// Scratch that lets launch_gemm_bits spread the contraction of a very small output (M <= 64 or so) over the CUs.
size_t gemm_bits_split_bytes(int64_t M, int64_t K, int64_t N);

// Digit operand whose rows are the C columns of src [R, C] (row stride ld), contraction over src's rows.  With
// detect_narrow the operand comes out in its one-digit form when every element is zero or a power of two within six
// binades of its column's largest (its flag word tells the product which form it got).
int launch_split_digits_columns(const float *src, int64_t ld, void *digits, int64_t R, int64_t C, bool detect_narrow,
                                hipStream_t stream);
// The statistics that pass gathers, kept in the operand's own row-sum area: per column the largest and the smallest
// non-zero magnitude (bit patterns, by atomicMax / atomicMin from 0 / 0xffffffff) and a flag word raised when an
// element is neither zero nor a normal power of two.  A kernel that touches every element of src anyway may fill them
// itself (clearing them first) and call the second half of the pass.
struct ColumnScratch {
  uint32_t *cmax, *cmin;
  int32_t *flag;
  int64_t rows; // entries of cmax / cmin (columns padded to whole fragments)
};
ColumnScratch column_scratch(void *digits, int64_t R, int64_t C);
int launch_split_digits_columns_from_stats(const float *src, int64_t ld, void *digits, int64_t R, int64_t C,
                                           bool detect_narrow, hipStream_t stream);
// y[m, n] (+)= sum_k A[m, k] * B[n, k] (+ bias[n]), both factors real-valued digit operands (rows M x K and N x K);
// A is a row-scaled operand, B a row- or column-scaled one whose flag word selects the six- or three-product form.
// `split_ws` (may be null; gemm_digits_split_bytes(M, K, N) bytes make every split possible) lets an output of few
// tiles with a long contraction spread the contraction over the CUs: dense partial results, summed in a fixed order.
int launch_gemm_digits(const void *adigits, const void *bdigits, const float *bias, float *y, int64_t M, int64_t K,
                       int64_t N, int64_t inner, int64_t outer_stride, int64_t n_stride, hipStream_t stream,
                       bool accumulate = false, void *split_ws = nullptr, size_t split_ws_bytes = 0);
size_t gemm_digits_split_bytes(int64_t M, int64_t K, int64_t N);

// BinaryWeightAffine / BinaryConnectAffine forward for very few input rows, in one pass over W [K, N] (no packed
// bits, no digit operand): writes Wb = Sign(W), alpha (when not null: alpha[n] = mean_k |W[k, n]|) and
// y = (x . Wb) (* alpha) (+ bias).  `applies` tells whether the shapes and alignments allow it.
constexpr int64_t kSmallMMaxRows = 16;  // rows the one-pass form multiplies on the vector ALUs
constexpr int64_t kFewRowsMaxRows = 64; // rows the one-pass form multiplies on the matrix cores
bool small_m_affine_applies(const float *x, const float *W, const float *Wb, const float *alpha, const float *bias,
                            const float *y, int64_t M, int64_t K, int64_t N, float zero_to);
size_t small_m_affine_workspace_bytes(int64_t M, int64_t K, int64_t N);
int launch_small_m_affine(const float *x, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                          int64_t M, int64_t K, int64_t N, float zero_to, void *workspace, size_t workspace_bytes,
                          hipStream_t stream);

// The same forward for up to kRowsMmaMaxRows input rows in one walk over W, on the int8 matrix cores
// (binary_rows_mma.hip): x comes as its digit operand (nbla_hip_split_digits_scaled_f32); rows marked kBadRow there are
// not written.  With zero_to other than +-1, *zero_flag (cleared by the caller) is raised when W holds a weight that
// is neither negative nor positive; y is then to be replaced by an fp32 product over Wb.  `workspace`
// (rows_affine_workspace_bytes, 16-byte aligned) holds the partial results when K is walked in slices.
constexpr int64_t kRowsMmaMaxRows = 512;
bool rows_affine_covers(const float *W, const float *Wb, const float *alpha, const float *bias, const float *y,
                        int64_t M, int64_t K, int64_t N);   // shapes it can run
bool rows_affine_pays(int64_t M, int64_t K, int64_t N);     // shapes on which it beats the two-walk path
size_t rows_affine_workspace_bytes(int64_t M, int64_t K, int64_t N);
int launch_rows_affine(const void *xdigits, const float *W, float *Wb, float *alpha, const float *bias, float *y,
                       int64_t M, int64_t K, int64_t N, float zero_to, int *zero_flag, void *workspace,
                       size_t workspace_bytes, hipStream_t stream);

// db[n] (+)= sum over m of dy[m, n]; `partial` holds ceil(M / 256) * N floats.
size_t column_sums_workspace_bytes(int64_t M, int64_t N);
int launch_column_sums(const float *dy, float *db, int64_t M, int64_t N, bool accumulate, void *partial,
                       hipStream_t stream);

} // namespace nbla_hip
