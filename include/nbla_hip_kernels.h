/*
 * nbla_hip_kernels.h -- C-ABI of the MI355X (gfx950) kernels behind nnabla's
 * quantization function family.
 *
 * Each entry point is what the `forward_impl` of a "hip:float" Function class
 * calls in place of the loop (or the chain of helper Functions) that nnabla's
 * CPU class runs; the reference interface it replaces is cited per function
 * (paths relative to the nnabla source tree).
 *
 * Conventions
 *   - plain C: raw DEVICE pointers, element counts, scalars; no C++/torch types.
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*;
 *     NULL = the default stream) unless its comment says it synchronises.
 *   - nothing here allocates device memory: scratch comes in through
 *     `workspace` arguments sized by the matching *_workspace_bytes() query.
 *     Workspaces must be 256-byte aligned.
 *   - return value: NBLA_HIP_OK (0); a negative NBLA_HIP_ERR_* for argument
 *     errors (mirroring nbla::error_code of the NBLA_CHECK the CPU class would
 *     raise); or a positive hipError_t.  nbla_hip_last_error() returns the
 *     message of the last failure on the calling thread.
 *   - all tensors are dense, C-contiguous fp32 unless stated otherwise.
 */
#ifndef NBLA_HIP_KERNELS_H_
#define NBLA_HIP_KERNELS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NBLA_HIP_OK 0
#define NBLA_HIP_ERR_NOT_IMPLEMENTED (-2) /* nbla::error_code::not_implemented */
#define NBLA_HIP_ERR_VALUE (-3)           /* nbla::error_code::value           */
#define NBLA_HIP_ERR_MEMORY (-5)          /* workspace too small / misaligned  */
#define NBLA_HIP_ERR_RUNTIME (-10)        /* library not initialised, bad arch */

/* ---------------------------------------------------------------- library */

/* Initialise the library for `device` (makes it current): checks that the
 * device is gfx950 and uploads the three per-binade cut tables that make
 * Pow2Quantize / INQ bit-exact against the host's libm (log2f is evaluated on
 * the host once per binade boundary, never per element).  Idempotent and
 * thread-safe; every other entry point calls it lazily for the current device.
 * Mirrors the role of init_cpu(): src/nbla/init.cpp.tmpl:44-111. */
int nbla_hip_init(int device);

const char *nbla_hip_last_error(void);
const char *nbla_hip_version(void);

/* Host-side view of the calibrated tables (277 uint32 entries each, indexed by
 * binade: subnormal binades 0..22, normal exponent field e at index e+22).
 * which: 0 = roundf(log2f(a)) (pow2_quantize.cpp:60), 1 = INQ weight exponent
 * (inq_affine.cpp:176-179), 2 = INQ n1 (inq_affine.cpp:161-164). */
int nbla_hip_cut_table(int which, uint32_t *out277);

/* ------------------------------------------------------ FixedPointQuantize */

/* y = FixedPointQuantize(x; sign, n, delta).
 * Replaces FixedPointQuantize<float>::forward_impl,
 * src/nbla/function/generic/fixed_point_quantize.cpp:46-66 (bounds from
 * setup_impl :29-43).  NBLA_HIP_ERR_VALUE when n <= 0, delta <= 0 or the
 * sign-adjusted width is <= 0, as the NBLA_CHECKs at :31-32 and :41-42.
 * In-place (y == x) is allowed. */
int nbla_hip_fixed_point_quantize_f32(const float *x, float *y, size_t size,
                                      int sign, int n, float delta,
                                      void *stream);

/* ------------------------------------------------------------ Pow2Quantize */

/* y = Pow2Quantize(x; sign, with_zero, n, m).
 * Replaces Pow2Quantize<float>::forward_impl,
 * src/nbla/function/generic/pow2_quantize.cpp:48-82 (setup :29-45).
 * NBLA_HIP_ERR_VALUE as the NBLA_CHECKs at :32 and :41-44;
 * NBLA_HIP_ERR_NOT_IMPLEMENTED when 2^m or 2^(m-(2^n'-1)) is not a finite
 * non-zero fp32 number. */
int nbla_hip_pow2_quantize_f32(const float *x, float *y, size_t size, int sign,
                               int with_zero, int n, int m, void *stream);

/* ---------------------------------------------------------- MinMaxQuantize */

/* Scratch for the min/max reduction partials and the nudged-range table. */
size_t nbla_hip_min_max_quantize_workspace_bytes(const int64_t *xshape,
                                                 int ndim,
                                                 const int64_t *qshape);

/* y = MinMaxQuantize(x, qr_min, qr_max, ql_min, ql_max; decay, x_min_max, ema,
 * eps).  Replaces MinMaxQuantize<float>::forward_impl,
 * src/nbla/function/generic/min_max_quantize.cpp:130-223 with nudge_range
 * (:353-361) and nudge_qr_min_max (:363-390): the ~20 helper-Function passes
 * become one min/max reduction (only when x_min_max) and one elementwise pass.
 * qshape has ndim entries, each 1 (reduced axis) or equal to xshape[i]; the four
 * q tensors and `scale` (the content of scale_sptr_, written) have that shape.
 * qr_min / qr_max are UPDATED IN PLACE exactly as the reference updates its
 * parameters.  NBLA_HIP_ERR_VALUE for a shape mismatch (:69-81). */
int nbla_hip_min_max_quantize_f32(const float *x, float *y,
                                  const int64_t *xshape, int ndim,
                                  const int64_t *qshape, float *qr_min,
                                  float *qr_max, const float *ql_min,
                                  const float *ql_max, float *scale,
                                  float decay, int x_min_max, int ema,
                                  float eps, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* The same forward for callers that cannot allocate device memory or carry a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  The reduction
 * partials and the nudged-range table live in a fixed array of
 * NBLA_HIP_STATIC_SCRATCH_BYTES inside the library, one copy per device, held
 * until the process ends; nbla_hip_init(device) must have run for the current
 * device (it resolves that device's copy), and the call itself allocates
 * nothing.  Shapes whose scratch (nbla_hip_min_max_quantize_workspace_bytes)
 * exceeds the array -- more than 8192 quantization ranges -- return
 * NBLA_HIP_ERR_MEMORY.  All calls on one device share the array: calls that
 * overlap on one device (different streams or threads) race; calls on one
 * stream are ordered.  Nothing in the array has to be cleared between calls
 * (every word read is written earlier in the same call).  Results are
 * bit-identical to nbla_hip_min_max_quantize_f32. */
#define NBLA_HIP_STATIC_SCRATCH_BYTES (256 * 1024)
int nbla_hip_min_max_quantize_static_f32(const float *x, float *y,
                                         const int64_t *xshape, int ndim,
                                         const int64_t *qshape, float *qr_min,
                                         float *qr_max, const float *ql_min,
                                         const float *ql_max, float *scale,
                                         float decay, int x_min_max, int ema,
                                         float eps, void *stream);

/* ------------------------------------------------ quantizers: backward (STE) */

/* dx (+)= dy inside [min, max], 0 outside (an accumulated dx is left alone
 * there); plain dx (+)= dy when ste_fine_grained == 0.  Replaces
 * FixedPointQuantize<float>::backward_impl,
 * src/nbla/function/generic/fixed_point_quantize.cpp:69-127.  accum != 0 adds to
 * the existing dx. */
int nbla_hip_fixed_point_quantize_backward_f32(const float *dy, const float *x,
                                               float *dx, size_t size, int sign,
                                               int n, float delta,
                                               int ste_fine_grained, int accum,
                                               void *stream);

/* dx (+)= c * dy with c = 0 where 2^round(log2|x|) > 2^m and, unsigned, where
 * x < 0.  Replaces Pow2Quantize<float>::backward_impl,
 * src/nbla/function/generic/pow2_quantize.cpp:84-156. */
int nbla_hip_pow2_quantize_backward_f32(const float *dy, const float *x,
                                        float *dx, size_t size, int sign,
                                        int with_zero, int n, int m,
                                        int ste_fine_grained, int accum,
                                        void *stream);

size_t nbla_hip_min_max_quantize_backward_workspace_bytes(const int64_t *xshape,
                                                          int ndim,
                                                          const int64_t *qshape);

/* Backward of MinMaxQuantize.  Replaces MinMaxQuantize<float>::backward_impl,
 * src/nbla/function/generic/min_max_quantize.cpp:225-350: with [m', M'] the
 * nudged range recomputed from qr_min, ql_min, ql_max and the forward's scale,
 *   dx       (+)= (x >= m') * (x <= M') * dy        (dy alone if not fine grained)
 *   g_qr_min (+)= sum over the reduced axes of (x < m') * dy
 *   g_qr_max (+)= sum over the reduced axes of (x > M') * dy
 * the range gradients only when neither x_min_max nor ema is set (:294-295).
 * dx, g_qr_min, g_qr_max may be NULL (not propagated). */
int nbla_hip_min_max_quantize_backward_f32(
    const float *dy, const float *x, float *dx, const int64_t *xshape, int ndim,
    const int64_t *qshape, const float *qr_min, const float *qr_max,
    const float *ql_min, const float *ql_max, const float *scale,
    float *g_qr_min, float *g_qr_max, int ste_fine_grained, int x_min_max,
    int ema, int accum_x, int accum_min, int accum_max, void *workspace,
    size_t workspace_bytes, void *stream);

/* ------------------------------------------- binary weights: sign/alpha/pack */

/* Bytes of the 1-bit packed GEMM operand for a [K, N] weight matrix (K padded
 * to 32, N to 256). */
size_t nbla_hip_packed_bits_bytes(int64_t K, int64_t N);
/* Bytes of the int8 digit operand for x [M, K] (the operand of the bit-weight
 * product): fragment-ordered digits, per-row sums and per-row shifts. */
size_t nbla_hip_digit_operand_bytes(int64_t M, int64_t K);
/* Scratch of nbla_hip_binarize_weights_f32 (column-sum partials, zero count). */
size_t nbla_hip_binarize_workspace_bytes(int64_t K, int64_t N);

/* Sign-binarise W and (optionally) compute alpha, in one pass over W:
 *   Wb[k,n]  = w>0 ? 1 : w<0 ? -1 : quantize_zero_to   (sign.hpp:48-50)
 *   alpha[n] = (sum_k |W[k,n]|) * ((float)1 / K)       (alpha may be NULL)
 *   bits     = 1 bit per weight (set = negative), in MFMA fragment order
 * The GEMM view is always B[k, n] with k the contraction index.
 *   transposed == 0: W is stored [K, N] (affine weights); replaces the
 *     Transpose/Abs/Sum/MulScalar/Sign passes of
 *     binary_weight_affine.cpp:85-102 and the Sign of
 *     binary_connect_affine.cpp:63-64.
 *   transposed == 1: W is stored [N, K] (convolution weights viewed
 *     [channels_o, col_w]); replaces binary_weight_convolution.cpp:83-98 and
 *     binary_connect_convolution.cpp:71-72.
 * Wb has W's own storage layout.  zero_count (device int, may be NULL) receives
 * the number of exact zeros in W: a non-zero count with quantize_zero_to other
 * than +-1 means `bits` alone cannot represent Wb. */
int nbla_hip_binarize_weights_f32(const float *W, float *Wb, float *alpha,
                                  uint32_t *bits, int64_t K, int64_t N,
                                  int transposed, float quantize_zero_to,
                                  int *zero_count, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* Turn x [M, K] (row stride ldx elements) into the int8 digit operand: per
 * row a power-of-two scale 2^s such that q = rint(x * 2^s) fits 24 bits for
 * the row's largest magnitude, q as three balanced base-256 digits in MFMA
 * fragment order, and the row sums of q.  A row holding NaN or infinity is
 * marked and yields NaN outputs. */
int nbla_hip_split_digits_f32(const float *x, int64_t ldx, void *xdigits,
                              int64_t M, int64_t K, void *stream);

/* Same, for the matrix x[m,k] * colscale[k] (one rounded fp32 product per
 * element; colscale may be NULL).  Used by the backward pass, where the
 * gradient is scaled by alpha before it meets the transposed binary weights. */
int nbla_hip_split_digits_scaled_f32(const float *x, int64_t ldx,
                                     const float *colscale, void *xdigits,
                                     int64_t M, int64_t K, void *stream);

/* y[m, n] = (sum_k x[m,k] * (+-1)[k,n]) * alpha[n] + bias[n]
 * with x given as the digit operand and the weights as packed bits; alpha and
 * bias may be NULL.  The sum is accumulated exactly in int32 on the int8 MFMA
 * units and converted to fp32 once, so it does not depend on summation order;
 * its error is the rounding of x to 24 bits relative to its row's largest
 * magnitude (K above 16384 is processed in chunks whose fp32 results are added).
 * Output addressing: element (m, n) is written at
 *   y[(m / inner) * outer_stride + n * n_stride + (m % inner)]
 * so a row-major [M, N] result is (inner=1, outer_stride=N, n_stride=1) and a
 * convolution result [batch, O, Ho*Wo] is (inner=Ho*Wo, outer_stride=O*Ho*Wo,
 * n_stride=Ho*Wo).  Replaces the Eigen product of affine.cpp:87-95 /
 * convolution.cpp:185-193 for binarised weights.
 * `workspace` (may be NULL; nbla_hip_gemm_bits_workspace_bytes(M, K, N) bytes,
 * 256-byte aligned) lets an output of very few tiles (M up to 64 or so) spread
 * its contraction over the CUs: fp32 partial results, summed in a fixed order. */
size_t nbla_hip_gemm_bits_workspace_bytes(int64_t M, int64_t K, int64_t N);
int nbla_hip_gemm_bits_f32(const void *xdigits, const uint32_t *bits,
                           const float *alpha, const float *bias, float *y,
                           int64_t M, int64_t K, int64_t N, int64_t inner,
                           int64_t outer_stride, int64_t n_stride,
                           void *workspace, size_t workspace_bytes,
                           void *stream);

/* ------------------------------------------------------- whole-op forwards */

size_t nbla_hip_binary_affine_workspace_bytes(int64_t M, int64_t K, int64_t N);

/* BinaryWeightAffine forward: x [M,K], W [K,N] -> Wb [K,N], alpha [N], y [M,N]
 * (bias [N] may be NULL).  Replaces BinaryWeightAffine<float>::forward_impl,
 * src/nbla/function/generic/binary_weight_affine.cpp:75-122.
 * The call never synchronises: when quantize_zero_to is neither +1 nor -1 the
 * weights that are neither negative nor positive are counted on the device, and
 * an fp32 product over the materialised signs Wb, launched behind the
 * matrix-core product with that count as its go-ahead, replaces y when the
 * count is non-zero (and leaves at once otherwise). */
int nbla_hip_binary_weight_affine_f32(const float *x, const float *W,
                                      float *Wb, float *alpha,
                                      const float *bias, float *y, int64_t M,
                                      int64_t K, int64_t N,
                                      float quantize_zero_to, void *workspace,
                                      size_t workspace_bytes, void *stream);

/* The same forward (alpha == NULL: BinaryConnectAffine) in its one-walk form,
 * whatever the shape: W is read once, by a kernel that writes Sign(W), sums |W|
 * per column and multiplies the fresh signs with the digit operand of x on the
 * int8 matrix cores (M <= 512, N % 4 == 0, W and Wb 16-byte aligned, K <= 16384,
 * W below 2 GiB; NBLA_HIP_ERR_NOT_IMPLEMENTED otherwise).  The two calls above
 * take this form by themselves for 65 <= M <= 256 on outputs wide enough to
 * occupy the CUs (strips of 128 columns x slices of K of at least 512 >= 128
 * blocks), where it is a fifth faster than two walks; this entry point is for
 * callers (and tests) that want it on other shapes.  Same reference functions,
 * same workspace. */
int nbla_hip_binary_affine_one_walk_f32(const float *x, const float *W,
                                        float *Wb, float *alpha,
                                        const float *bias, float *y, int64_t M,
                                        int64_t K, int64_t N,
                                        float quantize_zero_to, void *workspace,
                                        size_t workspace_bytes, void *stream);

size_t nbla_hip_affine_backward_workspace_bytes(int64_t M, int64_t K, int64_t N);

/* Backward of BinaryWeightAffine (alpha != NULL) / BinaryConnectAffine
 * (alpha == NULL): with Ws[k,n] = Sign(W)[k,n] * alpha[n] (or Sign(W)),
 *   dx[M,K] (+)= dy . Ws^T      dW[K,N] (+)= x^T . dy      db[N] (+)= sum_m dy
 * The weight gradient passes straight through the binarisation (Sign backward
 * is the identity, sign.hpp:48-50).  Replaces
 * BinaryWeightAffine<float>::backward_impl, binary_weight_affine.cpp:124-146,
 * BinaryConnectAffine<float>::backward_impl, binary_connect_affine.cpp:73-92
 * and the Affine backward they call, affine.cpp:98-140.  dx runs on the
 * bit-weight product (W is binarised again into its transposed packing); Wb
 * (the forward's fp32 signs) is only needed when quantize_zero_to is neither +1
 * nor -1, and only read when W then holds weights that are neither negative nor
 * positive: they are counted on the device, the bit-weight product does
 * nothing when the count is non-zero and an fp32 product over Wb launched
 * behind it does nothing when it is zero (no synchronisation, the host never
 * reads the count).  dx, dW, db may be NULL (not propagated); accum_* != 0 adds
 * to the existing gradient. */
int nbla_hip_binary_affine_backward_f32(const float *dy, const float *x,
                                        const float *W, const float *Wb,
                                        const float *alpha, float *dx,
                                        float *dW, float *db, int64_t M,
                                        int64_t K, int64_t N,
                                        float quantize_zero_to, int accum_x,
                                        int accum_w, int accum_b,
                                        void *workspace, size_t workspace_bytes,
                                        void *stream);

/* Backward of Affine with real-valued weights (the product inside INQAffine):
 *   dx (+)= dy . W^T      dW (+)= x^T . dy      db (+)= sum_m dy
 * Replaces Affine<float>::backward_impl, affine.cpp:98-140, as called by
 * INQAffine<float,int>::backward_impl, inq_affine.cpp:218-232. */
int nbla_hip_affine_backward_f32(const float *dy, const float *x, const float *W,
                                 float *dx, float *dW, float *db, int64_t M,
                                 int64_t K, int64_t N, int accum_x, int accum_w,
                                 int accum_b, void *workspace,
                                 size_t workspace_bytes, void *stream);

/* BinaryConnectAffine forward (no alpha).  Replaces
 * BinaryConnectAffine<float>::forward_impl,
 * src/nbla/function/generic/binary_connect_affine.cpp:60-71. */
int nbla_hip_binary_connect_affine_f32(const float *x, const float *W,
                                       float *Wb, const float *bias, float *y,
                                       int64_t M, int64_t K, int64_t N,
                                       float quantize_zero_to, void *workspace,
                                       size_t workspace_bytes, void *stream);

/* Plain fp32 GEMM y[M,N] = x[M,K] * w[K,N] (+ bias[N]) on the fp32 MFMA units.
 * Replaces Affine<float>::forward_impl, src/nbla/function/generic/affine.cpp:81-96. */
int nbla_hip_affine_f32(const float *x, const float *w, const float *bias,
                        float *y, int64_t M, int64_t K, int64_t N,
                        void *stream);

/* The same product on the int8 digit kernels (x row-scaled, w column-scaled,
 * three int8 digits each, six exact digit products per output; three when every
 * weight is zero or a power of two within six binades of its column's largest):
 * several times the fp32 MFMA rate at fp32-faithful accuracy (each operand is
 * rounded to 24 bits relative to its row / column maximum). */
size_t nbla_hip_affine_workspace_bytes(int64_t M, int64_t K, int64_t N);
int nbla_hip_affine_digits_f32(const float *x, const float *w, const float *bias,
                               float *y, int64_t M, int64_t K, int64_t N,
                               void *workspace, size_t workspace_bytes,
                               void *stream);

/* ------------------------------------------------------ binary convolutions */

/* Output spatial shape (i + 2p - (d(k-1)+1)) / s + 1 per dimension, as
 * Convolution<T>::setup_impl, src/nbla/function/generic/convolution.cpp:91-104.
 * NBLA_HIP_ERR_VALUE for a non-positive output size (the NBLA_CHECK at :99-103). */
int nbla_hip_convolution_output_shape(int nd, const int64_t *in_sp,
                                      const int64_t *kernel, const int64_t *pad,
                                      const int64_t *stride,
                                      const int64_t *dilation, int64_t *out_sp);

size_t nbla_hip_binary_convolution_workspace_bytes(
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, float quantize_zero_to);

/* Which form the binary convolutions' forward takes for a geometry, decided on
 * the host from the shapes alone (no counterpart in nnabla, whose one
 * forward_impl serves every geometry; for tests and for callers that want to
 * know).  plan[0] = output positions per block of the form that keeps the input
 * positions under a block in LDS (0: the geometry takes the gathering product),
 * plan[1] = blocks per sample, plan[2] = input positions the LDS of a block
 * holds, plan[3] = LDS bytes per block.  Touches no device. */
int nbla_hip_binary_convolution_slab_plan(
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, int32_t *plan);

/* BinaryWeightConvolution forward, channel-first, nd = 1..3 spatial dimensions:
 *   x [outer, C, in_sp...], W [O, C/group, kernel...] -> Wb (same shape as W),
 *   alpha [O], y [outer, O, out_sp...]; bias [O] may be NULL.
 * Replaces BinaryWeightConvolution<float>::forward_impl,
 * src/nbla/function/generic/binary_weight_convolution.cpp:73-117 (alpha per
 * output channel with the rounded reciprocal of col_w, :66) and the im2col +
 * per-sample Eigen product of convolution.cpp:161-197 / unfold_to_patches.cpp.
 * Argument errors as convolution.cpp:61-103.  A window of x that holds a NaN
 * or an infinity gives what the reference's product gives output by output
 * (+-Inf by the weight's sign, NaN for Inf - Inf): its outputs are recomputed
 * in fp32 over Wb.  Never synchronises: a
 * quantize_zero_to that is neither +1 nor -1 is handled on the device, as in
 * nbla_hip_binary_weight_affine_f32 (per group: unfold + fp32 product over Wb
 * behind the matrix-core product, with the group's count of weights that are
 * neither negative nor positive as their go-ahead). */
int nbla_hip_binary_weight_convolution_f32(
    const float *x, const float *W, float *Wb, float *alpha, const float *bias,
    float *y, int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, float quantize_zero_to,
    void *workspace, size_t workspace_bytes, void *stream);

/* BinaryConnectConvolution forward (no alpha).  Replaces
 * BinaryConnectConvolution<float>::forward_impl,
 * src/nbla/function/generic/binary_connect_convolution.cpp:68-80. */
int nbla_hip_binary_connect_convolution_f32(
    const float *x, const float *W, float *Wb, const float *bias, float *y,
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, float quantize_zero_to,
    void *workspace, size_t workspace_bytes, void *stream);

/* Convolution with real-valued weights, y = conv(x, W) + bias on the int8 digit
 * product (three digits per operand, exact int32 accumulation).  Replaces
 * Convolution<float>::forward_impl, convolution.cpp:161-197. */
size_t nbla_hip_convolution_workspace_bytes(
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group);
int nbla_hip_convolution_f32(const float *x, const float *W, const float *bias,
                             float *y, int64_t outer, int64_t C, int nd,
                             const int64_t *in_sp, int64_t O,
                             const int64_t *kernel, const int64_t *pad,
                             const int64_t *stride, const int64_t *dilation,
                             int64_t group, void *workspace,
                             size_t workspace_bytes, void *stream);

/* Workspace of the two convolution backward entry points below. */
size_t nbla_hip_convolution_backward_workspace_bytes(
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group);

/* Backward of BinaryWeightConvolution (alpha != NULL, alpha[o] scales output
 * channel o) / BinaryConnectConvolution (alpha == NULL): Convolution backward
 * with the weights Ws = Sign(W) (* alpha),
 *   dx (+)= fold(Ws_g^T . dy_g)    dW (+)= dy_g . unfold(x)_g^T    db (+)= sums of dy
 * the weight gradient passing straight through the binarisation.  Replaces
 * BinaryWeightConvolution<float>::backward_impl,
 * binary_weight_convolution.cpp:119-142,
 * BinaryConnectConvolution<float>::backward_impl,
 * binary_connect_convolution.cpp:83-103, the Convolution backward they call,
 * convolution.cpp:199-283, and fold_from_patches.cpp:95-170.  dy is
 * [outer, O, out_sp...], x [outer, C, in_sp...], W and dW [O, C/group, kernel...].
 * dx runs on the bit-weight product; Wb (the forward's fp32 signs) is only
 * needed when quantize_zero_to is neither +1 nor -1 and only read when W then
 * holds weights that are neither negative nor positive (decided on the device as
 * in nbla_hip_binary_affine_backward_f32: no synchronisation).  dx, dW, db may
 * be NULL (not propagated); accum_* != 0 adds to the existing gradient. */
int nbla_hip_binary_convolution_backward_f32(
    const float *dy, const float *x, const float *W, const float *Wb,
    const float *alpha, float *dx, float *dW, float *db, int64_t outer,
    int64_t C, int nd, const int64_t *in_sp, int64_t O, const int64_t *kernel,
    const int64_t *pad, const int64_t *stride, const int64_t *dilation,
    int64_t group, float quantize_zero_to, int accum_x, int accum_w,
    int accum_b, void *workspace, size_t workspace_bytes, void *stream);

/* Backward of Convolution with real-valued weights (the product inside
 * INQConvolution).  Replaces Convolution<float>::backward_impl,
 * convolution.cpp:199-283, as called by
 * INQConvolution<float,int>::backward_impl, inq_convolution.cpp:220-232. */
int nbla_hip_convolution_backward_f32(
    const float *dy, const float *x, const float *W, float *dx, float *dW,
    float *db, int64_t outer, int64_t C, int nd, const int64_t *in_sp,
    int64_t O, const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, int accum_x, int accum_w,
    int accum_b, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------ QuantizeLinear / DequantizeLinear / Prune */

#define NBLA_HIP_DTYPE_BYTE 1  /* nbla::dtypes::BYTE  (int8 range)  */
#define NBLA_HIP_DTYPE_UBYTE 2 /* nbla::dtypes::UBYTE (uint8 range) */

/* y = saturate(round(x / scale) + zp') with zp' = saturate(round(zero_point))
 * written back into zero_point, every step rounded in fp32 on its own;
 * round is std::round (half_to_even == 0, "HALF_AWAY_FROM_ZERO") or round-half-
 * to-even ("HALF_TO_EVEN"); the range is [-128,127] / [0,255] for BYTE / UBYTE,
 * [-127,127] / [1,255] with narrow_range.  scale and zero_point have x's number
 * of dimensions with each size 1 (broadcast) or equal to x's.  Replaces
 * QuantizeLinear<float>::forward_impl, quantize_linear.cpp:25-117 (setup checks
 * :28-46 -> NBLA_HIP_ERR_VALUE). */
int nbla_hip_quantize_linear_f32(const float *x, const float *scale,
                                 float *zero_point, float *y,
                                 const int64_t *xshape,
                                 const int64_t *scale_shape,
                                 const int64_t *zero_point_shape, int ndim,
                                 int half_to_even, int narrow_range, int dtype,
                                 void *stream);
/* dx (+)= dy / scale.  Replaces the x branch of
 * QuantizeLinear<float>::backward_impl, quantize_linear.cpp:119-156 (gradients
 * of scale and zero point are not_implemented there too). */
int nbla_hip_quantize_linear_backward_f32(const float *dy, const float *scale,
                                          float *dx, const int64_t *xshape,
                                          const int64_t *scale_shape, int ndim,
                                          int accum, void *stream);

/* y = (x - zero_point) * scale.  Replaces
 * DequantizeLinear<float>::forward_impl, dequantize_linear.cpp:25-67. */
int nbla_hip_dequantize_linear_f32(const float *x, const float *scale,
                                   const float *zero_point, float *y,
                                   const int64_t *xshape,
                                   const int64_t *scale_shape,
                                   const int64_t *zero_point_shape, int ndim,
                                   void *stream);
/* dx (+)= dy * scale.  dequantize_linear.cpp:69-108. */
int nbla_hip_dequantize_linear_backward_f32(const float *dy, const float *scale,
                                            float *dx, const int64_t *xshape,
                                            const int64_t *scale_shape,
                                            int ndim, int accum, void *stream);

/* Prune: y = (|x| < t) ? 0 : x with t = the (int)((size-1)*rate)-th smallest
 * |x| (+1 when rate == 1).  Replaces Prune<float>::forward_impl,
 * prune.cpp:27-70 (the full sort there is replaced by a radix select of that
 * one order statistic).  Its backward is the identity (prune.cpp:72-90):
 * use nbla_hip_fixed_point_quantize_backward_f32 with ste_fine_grained = 0.
 * The workspace (about 8 MiB, independent of size; contents need not be
 * cleared or kept between calls) holds the selection's histograms and the
 * candidate keys its second pass hands to its third. */
size_t nbla_hip_prune_workspace_bytes(void);
int nbla_hip_prune_f32(const float *x, float *y, size_t size, float rate,
                       void *workspace, size_t workspace_bytes, void *stream);

/* Range recorders of quantization-aware training: y = x (skipped when y == x)
 * and, when `training`, the one-element statistics m / M updated from this
 * batch.  Replaces the forward_impl of the five recorder PythonFunctions,
 * python/src/nnabla/utils/qnn.py:73-84 (mode 0, MinMaxMinMaxRecorder: m =
 * min(m, min x), M = max(M, max x)), :178-188 (1, AbsMaxRecorder: M = max(M,
 * max|x|)), :289-300 (2, MinMaxMvaRecorder: m = decay*m + (1-decay)*min x, M
 * likewise), :411-420 (3, MaxMaxRecorder) and :509-518 (4, MaxMvaRecorder); the
 * chains of Min / Max / Abs / Maximum2 / MulScalar / Add2 / Identity helper
 * functions there become one scan and one update.  `m` is unused in modes 1, 3
 * and 4.  `decay` is the Python float of the reference: decay and 1 - decay
 * are each rounded to fp32 once, as its MulScalar functions do.  Their backward passes the gradient through: use
 * nbla_hip_fixed_point_quantize_backward_f32 with ste_fine_grained = 0.
 * The launch elects its last block through counters in one of 16 slots inside
 * the library, handed out round-robin per process and put back to zero by that
 * block: at most 16 recorder launches may be in flight at once on one device
 * (on different streams; launches on one stream never overlap), and a launch
 * that is torn down part-way (device reset) leaves its slot unusable until the
 * library is loaded again. */
size_t nbla_hip_range_recorder_workspace_bytes(void);
int nbla_hip_range_recorder_f32(const float *x, float *y, size_t size, float *m,
                                float *M, int mode, double decay, int training,
                                void *workspace, size_t workspace_bytes,
                                void *stream);

/* Measurement aid; no counterpart in the reference.  After
 * nbla_hip_gemm_bits_timer_arm(n) the calling thread's next n launches of the
 * bit-weight product (by nbla_hip_gemm_bits_f32 or by the functions built on
 * it) each carry a pair of events that the runtime stamps with the dispatch's
 * own begin and end, so the kernel's duration is read as a profiler reads it,
 * without the queue bubbles of event records between launches.
 * nbla_hip_gemm_bits_timer_read waits for the launches made so far, returns
 * their number and the mean / smallest / largest duration in milliseconds and
 * disarms.  The results of the launches are unaffected. */
int nbla_hip_gemm_bits_timer_arm(int launches);
int nbla_hip_gemm_bits_timer_read(int *launches, double *mean_ms, double *min_ms,
                                  double *max_ms);

/* Measurement utility; no counterpart in the reference.  Launches a kernel of
 * nothing but independent matrix instructions on non-zero operands (two blocks
 * of four wavefronts per CU, `rounds` x 8 instructions per wavefront) so that
 * bench.py can time what the matrix pipes sustain under the part's power limit:
 * kind 0 = v_mfma_i32_32x32x32_i8, 1 = v_mfma_scale_f32_32x32x64_f8f6f4 with
 * fp6 x fp4 operands, 2 = the same with fp8 x fp8, 3 = the int8 instruction
 * with operands that change from one instruction to the next, 4 = as 3 with the
 * bit-weight product's operands (digits x bytes that are 0 or one power of
 * two).  Writes the number of instructions issued and the operations each one stands for; `sink` is a
 * device word that is never written. */
int nbla_hip_mfma_rate_probe(int kind, int rounds, int64_t *instructions,
                             int64_t *ops_per_instruction, float *sink,
                             void *stream);

/* ---------------------------------------------------------------------- INQ */

/* INQ step selector (what the forward does to the indicators before quantizing):
 *   -1  product only, weights untouched (recompute_impl, inq_affine.cpp:208-216)
 *    0  no selection this minibatch
 *    1  last entry of inq_iterations reached: every weight becomes fixed (:108-113)
 *    2  fix half of the learnable weights, largest |w| first (:117-141); equal |w|
 *       are taken in index order (the reference's order among equal keys is
 *       whatever std::sort leaves)
 *    3  fix each learnable weight with probability 1/2 (:143-149)
 * The caller owns the minibatch counter and maps it to a step. */

/* Bernoulli(0.5) source for step 3: must write `count` values (0 or 1) to `out`,
 * advancing the caller's generator by exactly `count` draws -- the role of
 * rdist_(rgen) with std::mt19937 in inq_affine.cpp:147. */
typedef void (*nbla_hip_bernoulli_fn)(void *ctx, uint8_t *out, int64_t count);

size_t nbla_hip_inq_workspace_bytes(int64_t size, int step);

/* Steps A, B, C and F of INQAffine<float,int>::forward_impl,
 * src/nbla/function/generic/inq_affine.cpp:95-190 and :203-204 (identical in
 * inq_convolution.cpp:110-222): W and I (int32 indicators) are rewritten in
 * place; old_W / old_I are the function's snapshot (read for the restore, then
 * overwritten with the new W / I).  n1n2_out (device, 2 ints, may be NULL)
 * receives the exponent range.  Step 3 synchronises the stream twice (the
 * number of learnable weights comes to the host, the host's draws go to the
 * device); every other step is asynchronous.  The same holds for the two
 * forwards below, which start with this update. */
int nbla_hip_inq_update_weights_f32(float *W, int32_t *I, float *old_W,
                                    int32_t *old_I, int64_t size, int num_bits,
                                    int step, nbla_hip_bernoulli_fn draw,
                                    void *draw_ctx, int32_t *n1n2_out,
                                    void *workspace, size_t workspace_bytes,
                                    void *stream);

size_t nbla_hip_inq_affine_workspace_bytes(int64_t M, int64_t K, int64_t N,
                                           int step);

/* INQAffine forward: the weight update above, then y = x . W + bias on the int8
 * digit product (exact int32 accumulation of digit products).  Replaces
 * INQAffine<float,int>::forward_impl, inq_affine.cpp:82-205. */
int nbla_hip_inq_affine_f32(const float *x, float *W, int32_t *I, float *old_W,
                            int32_t *old_I, const float *bias, float *y,
                            int64_t M, int64_t K, int64_t N, int num_bits,
                            int step, nbla_hip_bernoulli_fn draw,
                            void *draw_ctx, void *workspace,
                            size_t workspace_bytes, void *stream);

size_t nbla_hip_inq_convolution_workspace_bytes(
    int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
    const int64_t *kernel, const int64_t *pad, const int64_t *stride,
    const int64_t *dilation, int64_t group, int step);

/* INQConvolution forward.  Replaces INQConvolution<float,int>::forward_impl,
 * src/nbla/function/generic/inq_convolution.cpp:104-238. */
int nbla_hip_inq_convolution_f32(
    const float *x, float *W, int32_t *I, float *old_W, int32_t *old_I,
    const float *bias, float *y, int64_t outer, int64_t C, int nd,
    const int64_t *in_sp, int64_t O, const int64_t *kernel, const int64_t *pad,
    const int64_t *stride, const int64_t *dilation, int64_t group, int num_bits,
    int step, nbla_hip_bernoulli_fn draw, void *draw_ctx, void *workspace,
    size_t workspace_bytes, void *stream);

/* ------------------------------------------- device memory and array storage */

/* Thin wrappers the host layer (HipMemory, HipArray, the Hip backend singleton)
 * uses so that it needs no HIP headers: the counterparts of malloc/free in
 * src/nbla/memory/cpu_memory.cpp:49-80, of CpuArray::copy_from/zero/fill in
 * src/nbla/array/cpu_array.cpp and of BackendBase::device_synchronize
 * (include/nbla/backend_base.hpp:32-91).  `dtype` arguments are nbla::dtypes
 * codes (include/nbla/dtypes.hpp:32-64).  memcpy kind: 1 = host to device,
 * 2 = device to host (both complete before returning), 3 = device to device. */
int nbla_hip_get_device_count(int *count);
int nbla_hip_set_device(int device);
int nbla_hip_malloc(void **ptr, size_t bytes, int device);
int nbla_hip_free(void *ptr, int device);
int nbla_hip_mem_info(int device, size_t *free_bytes, size_t *total_bytes);
int nbla_hip_memcpy(void *dst, const void *src, size_t bytes, int kind,
                    void *stream);
int nbla_hip_device_synchronize(int device);
int nbla_hip_stream_synchronize(void *stream);
int nbla_hip_fill(void *dst, int dtype, size_t size, float value, void *stream);
int nbla_hip_cast(const void *src, int src_dtype, void *dst, int dst_dtype,
                  size_t size, void *stream);

/* y = x0 + x1 (same shapes).  Replaces Add2<float>::forward_impl,
 * src/nbla/function/generic/add2.cpp:39-47. */
int nbla_hip_add2_f32(const float *x0, const float *x1, float *y, size_t size,
                      void *stream);
/* dx (+)= dy.  Replaces add2_backward_cpu,
 * src/nbla/function/generic/add2.cpp:48-77. */
int nbla_hip_add2_backward_f32(const float *dy, float *dx, size_t size,
                               int accum, void *stream);
/* y = x0 - x1 (op 0), x0 * x1 (op 1), x0 / x1 (op 2) on inputs of one shape.
 * Replaces Sub2 / Mul2 / Div2 <float>::forward_impl: include/nbla/function/
 * sub2.hpp:41, mul2.hpp:42, div2.hpp:44 over utils/base_transform_binary.hpp:
 * 260-284. */
#define NBLA_HIP_BINARY2_SUB 0
#define NBLA_HIP_BINARY2_MUL 1
#define NBLA_HIP_BINARY2_DIV 2
int nbla_hip_binary2_f32(int op, const float *x0, const float *x1, float *y,
                         size_t size, void *stream);
/* dx = (accum ? dx : 0) + g with g the gradient of input `input` (0 or 1):
 * dy, -dy | dy * x1, dy * x0 | dy / x1, -dy * x0 / (x1 * x1).  Replaces
 * transform_binary_grad0 / grad1, utils/base_transform_binary.hpp:286-336,
 * with the gradient expressions of the headers above.  x0 and x1 are not
 * read for op 0. */
int nbla_hip_binary2_backward_f32(int op, int input, const float *dy,
                                  const float *x0, const float *x1, float *dx,
                                  size_t size, int accum, void *stream);
/* The same arithmetic with broadcasting, plus y = x0 + x1 (op 3) and the
 * element-wise power y = x0 ^ x1 (op 4: powf, dy x1 x0^(x1-1), dy log(x0) x0^x1;
 * include/nbla/function/pow2.hpp:44-47): shape0 and shape1 have `ndim` entries
 * each and differ only where one of them is 1; y has the larger size along
 * every axis.  Replaces BaseTransformBinary::setup_impl's shapes and strides and
 * transform_binary, utils/base_transform_binary.hpp:58-205 and :265-284 (Add2
 * reaches it through its BcAdd2 fall-back, add2.cpp:28-37).  Errors as :60-72.
 * The backward call gives dx = (accum ? dx : 0) + (the terms of every output
 * element the operand's element took part in), transform_binary_grad0 / grad1,
 * :286-336: for a broadcast operand a fixed-order parallel sum where the
 * reference adds one after the other in fp32 (equal to rounding, the same from
 * run to run).  With a workspace of nbla_hip_broadcast2_backward_workspace_bytes
 * (256-byte aligned; 0 bytes where the operand is not broadcast) the terms of
 * an element are spread over blocks; workspace NULL: one block per element of
 * the operand, whatever the number of its terms.  powf / logf are the device's,
 * not the host libm's: the power's bits are not pinned. */
#define NBLA_HIP_BINARY2_ADD 3
#define NBLA_HIP_BINARY2_POW 4
int nbla_hip_broadcast2_f32(int op, const float *x0, const int64_t *shape0,
                            const float *x1, const int64_t *shape1, float *y,
                            int ndim, void *stream);
int nbla_hip_broadcast2_backward_f32(int op, int input, const float *dy,
                                     const float *x0, const int64_t *shape0,
                                     const float *x1, const int64_t *shape1,
                                     float *dx, int ndim, int accum,
                                     void *workspace, size_t workspace_bytes,
                                     void *stream);
size_t nbla_hip_broadcast2_backward_workspace_bytes(int input,
                                                    const int64_t *shape0,
                                                    const int64_t *shape1,
                                                    int ndim);
/* dst[r * dst_stride + i] (+)= src[r * src_stride + i], r < rows, i < len:
 * one input's share of Concatenate<float>::forward_impl / backward_impl,
 * src/nbla/function/generic/concatenate.cpp:62-104 (rows = outer_size_, len =
 * the input's inner size, the other stride = inner_total_size_). */
int nbla_hip_copy_rows_f32(const float *src, int64_t src_stride, float *dst,
                           int64_t dst_stride, int64_t rows, int64_t len,
                           int accum, void *stream);

/* y = max(0, x).  Replaces ReLU<float>::forward_impl,
 * src/nbla/function/generic/relu.cpp (std::max(T(0), x)). */
int nbla_hip_relu_f32(const float *x, float *y, size_t size, void *stream);
/* dx (+)= (y > 0 ? dy : 0) with y the forward output.  Replaces
 * ReLU<float>::backward_impl, src/nbla/function/generic/relu.cpp:41-66. */
int nbla_hip_relu_backward_f32(const float *dy, const float *y, float *dx,
                               size_t size, int accum, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* NBLA_HIP_KERNELS_H_ */
