"""BinaryWeightAffine / BinaryConnectAffine on the GPU against the CPU oracle.

Bit-exact: Sign(W) (`Wb`) and the packed 1-bit operand.  At tolerance: alpha (rel 1e-6 against a float64
mean; the reference's own fp32 summation order comes from Eigen and is unpinned) and y
(max|y - y_ref| / max|y_ref| <= 1e-4 as the acceptance bar; the int8-digit product is expected below 1e-6).
"""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import unpack_digits, bits_equal, first_mismatch, max_rel_err, to_np, unpack_bits

pytestmark = pytest.mark.gpu

TOL = 1e-4         # north-star tolerance for GEMM outputs
TIGHT = 5e-6       # what an fp32-faithful product should reach on these sizes


def _dev(x, dev):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _data(M, K, N, seed=313, wscale=0.02):
    rng = np.random.RandomState(seed)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * wscale).astype(np.float32)
    return x, W


SHAPES = [(1, 32, 64), (2, 3, 4), (5, 17, 9), (8, 64, 64), (33, 100, 130), (64, 256, 256), (129, 96, 320),
          (300, 1000, 257), (7, 4096, 70), (1000, 200, 2100)]  # the last: 160 wide tiles, two k groups per block


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_binarize_bits_and_alpha(dev, M, K, N):
    _, W = _data(M, K, N)
    W.ravel()[::7] = 0.0            # exact zeros take quantize_zero_to
    W.ravel()[3::11] = -0.0
    for q0 in (1.0, -1.0):
        Wb, alpha, bits, zc = kernels.binarize_weights(_dev(W, dev), K, N, False, q0)
        ref_Wb, ref_alpha = oracle.binary_weight_prepare(W, q0)
        assert bits_equal(to_np(Wb), ref_Wb), first_mismatch(to_np(Wb), ref_Wb)
        unpacked = unpack_bits(to_np(bits), K, N)
        assert np.array_equal(unpacked, ref_Wb.astype(np.int8))
        a64 = np.abs(W.astype(np.float64)).mean(0)
        np.testing.assert_allclose(to_np(alpha), a64, rtol=2e-6, atol=1e-12)
        np.testing.assert_allclose(ref_alpha, a64, rtol=2e-6, atol=1e-12)
        assert int(to_np(zc)[0]) == int((W == 0).sum())


@pytest.mark.parametrize("K,N", [(9, 6), (2304, 256), (75, 130)])
def test_binarize_transposed_layout(dev, K, N):
    """Convolution weights are stored [N(out channels), K]; bits must equal the [K, N] view's."""
    rng = np.random.RandomState(1)
    Wnk = (rng.randn(N, K) * 0.03).astype(np.float32)
    Wnk.ravel()[::13] = 0.0
    Wb, alpha, bits, zc = kernels.binarize_weights(_dev(Wnk, dev), K, N, True, 1.0)
    ref_Wb = oracle.sign(Wnk, 1.0)
    assert bits_equal(to_np(Wb), ref_Wb)
    assert np.array_equal(unpack_bits(to_np(bits), K, N), ref_Wb.T.astype(np.int8))
    np.testing.assert_allclose(to_np(alpha), np.abs(Wnk.astype(np.float64)).mean(1), rtol=2e-6)


@pytest.mark.parametrize("M,K", [(45, 70), (45, 128), (64, 64), (100, 1024), (37, 2048), (1, 4096), (19, 5000), (33, 8192),
                                 (21, 11008), (9, 16384), (3, 16384 + 40)])
def test_digit_operand(dev, M, K):
    """The int8 digit operand: q = rint(x * 2^s) with the largest power-of-two scale that keeps the row inside three
    balanced base-256 digits, digits in fragment order, exact row sums per k chunk (rows of up to 16384 values with
    K % 4 == 0 take the one-pass kernel in its eight shapes, the others the two-pass kernels)."""
    rng = np.random.RandomState(2)
    x = (rng.randn(M, K) * np.exp(rng.randn(M, 1) * 8)).astype(np.float32)
    x[0, :6] = [0.0, -0.0, 1e-30, -3e-5, 3.3e-7, 1.0]
    if M > 2:
        x[2] = 0.0
    q, shift, sums = unpack_digits(to_np(kernels.split_digits(_dev(x, dev), M, K)), M, K)
    x64 = x.astype(np.float64)
    expect = np.rint(np.ldexp(x64, shift[:, None].astype(np.int64)))          # exact scaling, ties to even
    assert np.array_equal(q, expect.astype(np.int64))
    amax = np.abs(q).max(1)
    assert (amax <= 8355711).all()
    nz = np.abs(x).max(1) > 0
    # the scale is maximal: one more doubling would leave the digit range
    assert (np.rint(np.ldexp(np.abs(x64).max(1)[nz], shift[nz].astype(np.int64) + 1)) > 8355711).all()
    assert (shift[~nz] == 0).all()
    for c in range(sums.shape[0]):
        assert np.array_equal(sums[c], q[:, c * 16384:(c + 1) * 16384].sum(1))
    # value error: at most half a unit of the row's scale
    assert (np.abs(np.ldexp(q.astype(np.float64), -shift[:, None].astype(np.int64)) - x64)
            <= np.ldexp(0.5, -shift[:, None].astype(np.int64))).all()


@pytest.mark.parametrize("M,K", [(4100, 128), (4100, 512), (4100, 2048), (2100, 64), (2100, 4096), (2100, 6000),
                                 (2100, 8192), (2100, 11008), (1100, 4096), (1100, 100)])
def test_digit_operand_block_shapes(dev, M, K):
    """Row counts that give every CU a block select the one-pass kernel's 16- and 8-row shapes; the operand must not
    depend on the shape."""
    rng = np.random.RandomState(M + K)
    x = (rng.randn(M, K) * np.exp(rng.randn(M, 1) * 4)).astype(np.float32)
    x[5] = 0.0
    x[7, K // 2] = np.inf
    q, shift, sums = unpack_digits(to_np(kernels.split_digits(_dev(x, dev), M, K)), M, K)
    assert shift[7] == -2 ** 31 and not q[7].any() and sums[0, 7] == 0 and shift[5] == 0
    ok = np.ones(M, bool)
    ok[7] = False
    amax = np.abs(x[ok]).max(1).astype(np.float64)
    want = np.where(amax > 0, 22 - np.floor(np.log2(np.where(amax > 0, amax, 1.0))), 0).astype(np.int64)
    want -= (np.rint(np.ldexp(amax, want)) > 8355711)
    assert np.array_equal(shift[ok], want)
    assert np.array_equal(q[ok], np.rint(np.ldexp(x[ok].astype(np.float64), want[:, None])).astype(np.int64))
    assert np.array_equal(sums[0], q.sum(1))


@pytest.mark.parametrize("M,K,ldx", [(70, 256, 260), (2100, 1024, 1100), (33, 4096, 4100), (40, 90, 97), (64, 8192, 8200)])
def test_digit_operand_of_a_strided_matrix(dev, M, K, ldx):
    """Row stride larger than the row length (a slice of a wider matrix): the operand only depends on the M x K view."""
    rng = np.random.RandomState(K)
    wide = rng.randn(M, ldx).astype(np.float32)
    view = np.ascontiguousarray(wide[:, :K])
    a = to_np(kernels.split_digits(_dev(wide, dev), M, K, ldx=ldx))
    b = to_np(kernels.split_digits(_dev(view, dev), M, K))
    qa, sa, ma = unpack_digits(a, M, K)
    qb, sb, mb = unpack_digits(b, M, K)
    assert np.array_equal(qa, qb) and np.array_equal(sa, sb) and np.array_equal(ma, mb)
    assert np.array_equal(qa, np.rint(np.ldexp(view.astype(np.float64), sa[:, None].astype(np.int64))).astype(np.int64))


def test_digit_operand_marks_non_finite_rows(dev):
    x = np.ones((40, 64), np.float32)
    x[1, 3] = np.inf
    x[3, 60] = np.nan
    W = np.ones((64, 64), np.float32)
    _, shift, _ = unpack_digits(to_np(kernels.split_digits(_dev(x, dev), 40, 64)), 40, 64)
    assert shift[1] == -2 ** 31 and shift[3] == -2 ** 31 and shift[0] == shift[2] == shift[4]
    # the whole function: marked rows are recomputed element by element, as the reference's product leaves them
    y, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))      # 40 rows: the digit-operand product
    y = to_np(y)
    ok = np.ones(40, bool)
    ok[[1, 3]] = False
    assert np.isposinf(y[1]).all() and np.isnan(y[3]).all()
    assert np.array_equal(y[ok], np.full((38, 64), 64.0, np.float32))
    # the product alone leaves NaN in a marked row
    _, _, bits, _ = kernels.binarize_weights(_dev(W, dev), 64, 64, want_alpha=False)
    yp = to_np(kernels.gemm_bits(kernels.split_digits(_dev(x, dev), 40, 64), bits, None, None, 40, 64, 64))
    assert np.isnan(yp[[1, 3]]).all() and np.array_equal(yp[ok], y[ok])


@pytest.mark.parametrize("weight", [True, False])
@pytest.mark.parametrize("M,K,N", [(70, 96, 130),      # few tiles: the contraction is spread over blocks and summed
                                   (70, 98, 130),      # rows that are no multiple of four values: two-pass digit split
                                   (300, 256, 600)])   # wide tiles, edge columns
def test_many_rows_propagate_non_finite_values_per_element(dev, weight, M, K, N):
    """Above sixteen rows the product runs on integer digits; rows holding Inf / NaN are recomputed in fp32 (by the
    kernel that splits x into digits, or after the product where that kernel is the two-pass form) so that every
    output element is what the reference's product gives (affine.cpp:87-95)."""
    rng = np.random.RandomState(12)
    x = rng.randn(M, K).astype(np.float32)
    x[1, 3] = np.inf
    x[2, 7], x[2, 9] = -np.inf, np.inf
    x[40, 60] = np.nan
    x[69, 0] = -np.inf
    W = rng.randn(K, N).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    if weight:
        y, _, _ = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
        ref, _, _ = oracle.binary_weight_affine(x, W, b, 1.0)
    else:
        y, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
        ref, _ = oracle.binary_connect_affine(x, W, b, 1.0)
    y = to_np(y)
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin.sum() >= (M - 4) * N and np.abs(y[fin] - ref[fin]).max() <= 1e-4 * np.abs(ref[fin]).max()


def test_few_rows_propagate_non_finite_values_per_element(dev):
    """The one-pass product for a handful of rows multiplies and adds in fp32, so Inf and NaN spread exactly as in
    the reference's product (affine.cpp:87-95): per output element."""
    rng = np.random.RandomState(11)
    x = rng.randn(5, 64).astype(np.float32)
    x[1, 3] = np.inf
    x[2, 7] = -np.inf
    x[2, 9] = np.inf
    x[3, 60] = np.nan
    W = rng.randn(64, 64).astype(np.float32)
    y, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))
    y = to_np(y)
    ref, _ = oracle.binary_connect_affine(x, W, None, 1.0)
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin[[0, 4]].all() and np.abs(y[fin] - ref[fin]).max() <= 1e-4 * np.abs(ref[fin]).max()
    assert np.isinf(y[1]).all() and np.isnan(y[3]).all()


@pytest.mark.parametrize("M", [9, 16, 17, 32, 33, 50, 64])
@pytest.mark.parametrize("K,N", [(304, 1028), (256, 256), (1008, 516), (64, 4), (4112, 260), (16, 132)])
def test_some_dozen_rows_one_pass_product_on_the_matrix_cores(dev, M, K, N):
    """9 <= M <= 64 with K % 16 == 0 and N % 4 == 0 also runs in one walk over W: the signs go straight from the
    registers into bf16 matrix instructions, against x split exactly into three bf16 terms.  Ragged strips of N,
    tile counts that leave wavefronts and slabs short, both row-fragment counts, rows that stop inside a fragment;
    Wb bit-exact, alpha and y against the oracle and float64.  Weights include exact zeros of both signs and a NaN
    (Sign -> zero_to)."""
    x, W = _data(M, K, N, seed=M * 1000 + K)
    W.ravel()[::7] = 0.0
    W.ravel()[3::11] = -0.0
    W[K // 2, N // 2] = np.nan
    b = np.random.RandomState(2).randn(N).astype(np.float32)
    for q0 in (1.0, -1.0, 0.0, 0.5):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, q0)
        y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev), q0)
        assert bits_equal(to_np(Wb), ref_Wb), first_mismatch(to_np(Wb), ref_Wb)
        col_ok = ~np.isnan(ref_alpha)                       # the NaN weight's column has a NaN mean in both
        assert np.array_equal(np.isnan(to_np(alpha)), ~col_ok)
        np.testing.assert_allclose(to_np(alpha)[col_ok], ref_alpha[col_ok], rtol=2e-6)
        assert max_rel_err(to_np(y)[:, col_ok], ref_y[:, col_ok]) <= TIGHT * 4
        assert np.isnan(to_np(y)[:, ~col_ok]).all()
        ref_y, ref_Wb = oracle.binary_connect_affine(x, W, None, q0)
        y, Wb = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev), None, q0)
        assert bits_equal(to_np(Wb), ref_Wb)
        y64 = x.astype(np.float64) @ ref_Wb.astype(np.float64)
        assert max_rel_err(to_np(y), y64) <= TIGHT and max_rel_err(to_np(y), ref_y) <= TIGHT * 4


def test_some_dozen_rows_keep_every_bit_of_x(dev):
    """The three bf16 terms carry all 24 significand bits: with weights of one sign the product is the plain sum of a
    row of x, and inputs chosen so that every partial sum is exact in fp32 (integers below 2^24 scaled by a power of
    two, including values that need all three terms and values whose lower terms are zero) must come out exactly."""
    M, K, N = 40, 64, 8
    rng = np.random.RandomState(5)
    ints = rng.randint(-(1 << 17), 1 << 17, size=(M, K)).astype(np.int64)
    ints[:, 0] = (1 << 17) - 1                                   # seventeen ones: all three terms in use
    ints[:, 1] = 1 << 16                                         # one bit: the lower terms are zero
    ints[:, 2] = -((1 << 17) - 1)
    ints[3, :] = 0
    x = (ints.astype(np.float64) * 2.0 ** -20).astype(np.float32)
    W = np.full((K, N), 0.25, np.float32)
    W[:, 1::2] = -0.25
    y, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))
    want = (ints.sum(1).astype(np.float64) * 2.0 ** -20)[:, None] * np.where(np.arange(N) % 2 == 0, 1.0, -1.0)
    assert np.array_equal(to_np(y).astype(np.float64), want)


def test_some_dozen_rows_propagate_non_finite_values_per_element(dev):
    """Inf and NaN stay in the first of the three bf16 terms of x (also a NaN whose payload lies in the lower half of
    the word), so they spread per output element exactly as in the reference's fp32 product (affine.cpp:87-95)."""
    rng = np.random.RandomState(13)
    M, K, N = 40, 64, 64
    x = rng.randn(M, K).astype(np.float32)
    x[1, 3] = np.inf
    x[2, 7], x[2, 9] = -np.inf, np.inf
    x[3, 60] = np.nan
    x.view(np.uint32)[4, 5] = 0x7f800001                          # signalling NaN, payload in the low bits only
    x[35, 0] = -np.inf
    x[36, 1] = 3.0e38
    x[36, 2] = 3.0e38                                             # finite inputs whose sum overflows
    W = rng.randn(K, N).astype(np.float32)
    W[1, :], W[2, :] = 1.0, 1.0
    y, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))
    y = to_np(y)
    with np.errstate(over="ignore", invalid="ignore"):
        ref, _ = oracle.binary_connect_affine(x, W, None, 1.0)
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin[[0, 5, 39]].all() and np.abs(y[fin] - ref[fin]).max() <= 1e-4 * np.abs(ref[fin]).max()
    assert np.isinf(y[1]).all() and np.isnan(y[3]).all() and np.isnan(y[4]).all() and np.isposinf(y[36]).all()


@pytest.mark.parametrize("M,K,N", [(3, 16384 + 40, 70), (40, 40000, 64)])
def test_long_contraction_is_chunked(dev, M, K, N):
    """K above 16384 is accumulated in int32 per chunk of 16384 columns and the chunks are added in fp32."""
    x, W = _data(M, K, N, seed=3)
    b = np.random.RandomState(4).randn(N).astype(np.float32)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
    sgn = np.where(W >= 0, 1.0, -1.0)
    y64 = x.astype(np.float64) @ (sgn * np.abs(W.astype(np.float64)).mean(0)) + b
    assert max_rel_err(to_np(y), y64) <= TIGHT


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("bias", [False, True])
def test_binary_weight_affine_matches_oracle(dev, M, K, N, bias):
    x, W = _data(M, K, N)
    b = np.random.RandomState(9).randn(N).astype(np.float32) if bias else None
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, 1.0)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), None if b is None else _dev(b, dev))
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    y64 = x.astype(np.float64) @ (ref_Wb.astype(np.float64) * np.abs(W.astype(np.float64)).mean(0))
    if b is not None:
        y64 = y64 + b
    assert max_rel_err(to_np(y), ref_y) <= TOL
    assert max_rel_err(to_np(y), y64) <= TIGHT
    assert max_rel_err(ref_y, y64) <= TIGHT


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_binary_connect_affine_matches_oracle(dev, M, K, N):
    x, W = _data(M, K, N, seed=7)
    b = np.random.RandomState(3).randn(N).astype(np.float32)
    ref_y, ref_Wb = oracle.binary_connect_affine(x, W, b, 1.0)
    y, Wb = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
    assert bits_equal(to_np(Wb), ref_Wb)
    y64 = x.astype(np.float64) @ ref_Wb.astype(np.float64) + b
    assert max_rel_err(to_np(y), ref_y) <= TOL
    assert max_rel_err(to_np(y), y64) <= TIGHT


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 9, 16])
@pytest.mark.parametrize("K,N", [(300, 1028), (256, 256), (1000, 516), (64, 4), (4097, 260)])
def test_few_rows_one_pass_product(dev, M, K, N):
    """M <= 16 with N % 4 == 0 runs the one-pass form (signs, column sums and dot products in a single walk over W):
    ragged last slab of K, ragged last strip of N, every row count the templates round up from; Wb bit-exact, alpha
    and y against the oracle and float64.  Weights include exact zeros of both signs and a NaN (Sign -> zero_to)."""
    x, W = _data(M, K, N, seed=M * 1000 + K)
    W.ravel()[::7] = 0.0
    W.ravel()[3::11] = -0.0
    W[K // 2, N // 2] = np.nan
    b = np.random.RandomState(2).randn(N).astype(np.float32)
    for q0 in (1.0, -1.0, 0.0, 0.5):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, q0)
        y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev), q0)
        assert bits_equal(to_np(Wb), ref_Wb), first_mismatch(to_np(Wb), ref_Wb)
        col_ok = ~np.isnan(ref_alpha)                       # the NaN weight's column has a NaN mean in both
        assert np.array_equal(np.isnan(to_np(alpha)), ~col_ok)
        np.testing.assert_allclose(to_np(alpha)[col_ok], ref_alpha[col_ok], rtol=2e-6)
        assert max_rel_err(to_np(y)[:, col_ok], ref_y[:, col_ok]) <= TIGHT * 4
        assert np.isnan(to_np(y)[:, ~col_ok]).all()
        ref_y, ref_Wb = oracle.binary_connect_affine(x, W, None, q0)
        y, Wb = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev), None, q0)
        assert bits_equal(to_np(Wb), ref_Wb)
        y64 = x.astype(np.float64) @ ref_Wb.astype(np.float64)
        assert max_rel_err(to_np(y), y64) <= TIGHT and max_rel_err(to_np(y), ref_y) <= TIGHT * 4


@pytest.mark.parametrize("M", [1, 33, 65, 100, 128, 200, 256, 257, 300, 512])
@pytest.mark.parametrize("K,N", [(96, 64), (100, 132), (256, 260), (1000, 516), (4100, 68), (32, 4)])
def test_one_walk_product_on_the_matrix_cores(dev, M, K, N):
    """The form that serves 65 <= M <= 512 on wide outputs -- one walk over W that writes Sign(W), sums |W| and
    multiplies the fresh signs with the digit operand of x on the int8 matrix cores -- called directly so that narrow
    and ragged shapes reach it too: ragged last k step, ragged last strip of 64 columns, both tile heights (256 and
    512 rows), wavefronts with no rows.  Weights include exact zeros of both signs and a NaN (Sign -> zero_to); Wb
    bit-exact, alpha and y against the oracle and float64, for every quantize_zero_to class (+-1: sign bits; other
    values: the fp32 product behind the device-side flag)."""
    x, W = _data(M, K, N, seed=M * 1000 + K)
    W.ravel()[::7] = 0.0
    W.ravel()[3::11] = -0.0
    W[K // 2, N // 2] = np.nan
    b = np.random.RandomState(2).randn(N).astype(np.float32)
    for q0 in (1.0, -1.0, 0.0, 0.3):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, q0)
        y, Wb, alpha = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), _dev(b, dev), q0)
        assert bits_equal(to_np(Wb), ref_Wb), first_mismatch(to_np(Wb), ref_Wb)
        col_ok = ~np.isnan(ref_alpha)                       # the NaN weight's column has a NaN mean in both
        assert np.array_equal(np.isnan(to_np(alpha)), ~col_ok)
        np.testing.assert_allclose(to_np(alpha)[col_ok], ref_alpha[col_ok], rtol=2e-6)
        assert max_rel_err(to_np(y)[:, col_ok], ref_y[:, col_ok]) <= TIGHT * 4
        assert np.isnan(to_np(y)[:, ~col_ok]).all()
        ref_y, ref_Wb = oracle.binary_connect_affine(x, W, None, q0)
        y, Wb, _ = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), None, q0, weight=False)
        assert bits_equal(to_np(Wb), ref_Wb)
        y64 = x.astype(np.float64) @ ref_Wb.astype(np.float64)
        assert max_rel_err(to_np(y), y64) <= TIGHT and max_rel_err(to_np(y), ref_y) <= TIGHT * 4


def test_one_walk_product_without_exact_zero_weights_keeps_the_matrix_core_result(dev):
    """quantize_zero_to = 0.3 on weights none of which is zero: the device-side flag stays down, the fp32 product
    leaves at once and y is the matrix-core result bit for bit (that of quantize_zero_to = 1)."""
    x, W = _data(130, 256, 200, seed=5)
    assert (W != 0).all()
    y1, Wb1, _ = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), None, 1.0)
    y3, Wb3, _ = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), None, 0.3)
    assert bits_equal(to_np(Wb1), to_np(Wb3)) and bits_equal(to_np(y1), to_np(y3))


def test_one_walk_product_propagates_non_finite_values_per_element(dev):
    rng = np.random.RandomState(12)
    M, K, N = 300, 256, 600
    x = rng.randn(M, K).astype(np.float32)
    x[1, 3] = np.inf
    x[2, 7], x[2, 9] = -np.inf, np.inf
    x[40, 60] = np.nan
    x[299, 0] = -np.inf
    W = rng.randn(K, N).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    y, _, _ = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), _dev(b, dev))
    ref, _, _ = oracle.binary_weight_affine(x, W, b, 1.0)
    y = to_np(y)
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin.sum() >= (M - 4) * N and np.abs(y[fin] - ref[fin]).max() <= 1e-4 * np.abs(ref[fin]).max()


def test_one_walk_product_refuses_what_it_does_not_cover(dev):
    x, W = _data(600, 64, 64)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev))
    assert ei.value.code == kernels.ERR_NOT_IMPLEMENTED
    x, W = _data(100, 64, 66)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev))
    assert ei.value.code == kernels.ERR_NOT_IMPLEMENTED


@pytest.mark.parametrize("M,K,N", [(100, 1024, 8196),   # 65 strips of 128 columns, K in two slices
                                   (256, 40, 16388),    # 129 strips, one short slice
                                   (65, 1600, 5640)])   # 45 strips, K in three slices
def test_wide_outputs_of_some_hundred_rows_take_the_one_walk_form(dev, M, K, N):
    """For 65..256 rows the whole-operation entry points run the one-walk form when its blocks (strips of 128 columns
    x slices of K) number at least 128; checked against the oracle like the other paths, and bit-identical to the
    direct call."""
    x, W = _data(M, K, N, seed=31)
    W.ravel()[::13] = 0.0
    b = np.random.RandomState(9).randn(N).astype(np.float32)
    for q0 in (1.0, 0.0):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, q0)
        y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev), q0)
        assert bits_equal(to_np(Wb), ref_Wb)
        np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
        assert max_rel_err(to_np(y), ref_y) <= TIGHT * 4
    y1, Wb1, a1 = kernels.binary_affine_one_walk(_dev(x, dev), _dev(W, dev), _dev(b, dev), 0.0)
    assert bits_equal(to_np(y1), to_np(y)) and bits_equal(to_np(a1), to_np(alpha))


@pytest.mark.parametrize("ratio_log2", [8, 12, 17])
@pytest.mark.parametrize("M", [8, 48, 200, 600])   # vector ALUs (no digits: control), bf16 terms, one walk, two walks
def test_error_bound_with_a_wide_range_inside_a_row(dev, M, ratio_log2):
    """The digit product rounds x to 24 bits relative to the largest magnitude OF ITS ROW (q = rint(x 2^s), 2^s the
    largest power of two with |q| <= 8355711), exactly once; everything after that is exact integer arithmetic and one
    rounding of the result.  So for every output
        |y - y64| <= K * max|x_row| / 8355711 * alpha + 2^-23 |y64|,
    whatever the values (typically sqrt(K) instead of K).  Rows with one or two outliers 2^8 .. 2^17 times the rest:
    where two outliers cancel in an output, that output's RELATIVE error can reach ratio * 2^-24 * O(1) -- a per cent
    at 2^17 -- where an fp32 sum in k order may be exact; relative to the largest output of the row (the metric of the
    acceptance bar, max|y - ref| / max|ref|) it stays below 2e-5.  The forms that do not use digits (up to 64 rows)
    split x into three bf16 terms or multiply in fp32 and are not subject to the bound; they are checked against the
    same figures."""
    K, N = 4096, 256
    rng = np.random.RandomState(100 + ratio_log2)
    x = rng.randn(M, K).astype(np.float32)
    big = np.float32(2.0 ** ratio_log2)
    kinds = np.arange(M) % 4                       # 0: plain row, 1: one outlier, 2: two that cancel where the signs
    for m in range(M):                             # agree, 3: two of the same sign
        j, k = rng.choice(K, 2, replace=False)
        if kinds[m] >= 1:
            x[m, j] = big * (1 + rng.rand())
        if kinds[m] == 2:
            x[m, k] = -x[m, j]
        if kinds[m] == 3:
            x[m, k] = x[m, j] * np.float32(0.75)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev))
    y, alpha = to_np(y).astype(np.float64), to_np(alpha).astype(np.float64)
    y64 = x.astype(np.float64) @ (np.sign(W).astype(np.float64) * alpha)
    row_max = np.abs(x).max(1).astype(np.float64)
    bound = K * row_max[:, None] / 8355711.0 * alpha[None, :] + 2.0 ** -23 * np.abs(y64)
    err = np.abs(y - y64)
    assert (err <= bound).all(), "worst err / bound = %.3g" % (err / bound).max()
    # what it means in the two metrics
    per_row = err.max(1) / np.abs(y64).max(1)
    rel = err / np.maximum(np.abs(y64), 1e-30)
    print("M=%d ratio 2^%d: err/bound max %.3g; err / max|y_row| max %.3g; per-element relative error max %.3g "
          "(rows with cancelling outliers: %.3g)" % (M, ratio_log2, (err / bound).max(), per_row.max(), rel.max(),
                                                      rel[kinds == 2].max()))
    assert per_row.max() <= 2e-5
    assert err.max() / np.abs(y64).max() <= 2e-5


@pytest.mark.parametrize("M,K,N", [(3100, 96, 5732), (3072, 64, 11008)])
def test_tall_m_every_element(dev, M, K, N):
    """Tall outputs with a ragged last column tile (idle wavefronts, clamped wide groups): every output element is
    checked against float64."""
    x, W = _data(M, K, N, seed=21)
    b = np.random.RandomState(5).randn(N).astype(np.float32)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
    sgn = np.where(W >= 0, 1.0, -1.0)
    assert bits_equal(to_np(Wb), sgn.astype(np.float32))
    y64 = x.astype(np.float64) @ (sgn * np.abs(W.astype(np.float64)).mean(0)) + b
    assert max_rel_err(to_np(y), y64) <= TIGHT
    yc, _ = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))
    assert max_rel_err(to_np(yc), x.astype(np.float64) @ sgn) <= TIGHT


@pytest.mark.parametrize("q0", [0.0, 0.5, -1.0, 1.0])
def test_quantize_zero_to_with_exact_zero_weights(dev, q0):
    """Sign(0) = quantize_zero_to (test_binary_weight_affine.py:72 covers 0, -1, 1)."""
    x, W = _data(40, 96, 72, seed=11)
    W.ravel()[::5] = 0.0
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, None, q0)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), None, q0)
    assert bits_equal(to_np(Wb), ref_Wb)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT * 4
    ref_y, ref_Wb = oracle.binary_connect_affine(x, W, None, q0)
    y, Wb = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev), None, q0)
    assert bits_equal(to_np(Wb), ref_Wb)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT * 4


def test_plain_affine_f32(dev):
    for (M, K, N) in [(2, 3, 4), (70, 130, 200), (256, 512, 384)]:
        x, W = _data(M, K, N, seed=5, wscale=1.0)
        b = np.random.RandomState(4).randn(N).astype(np.float32)
        y = to_np(kernels.affine(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
        y64 = x.astype(np.float64) @ W.astype(np.float64) + b
        assert max_rel_err(y, y64) <= TIGHT
        assert max_rel_err(oracle.affine(x, W, b), y64) <= TIGHT
        # the same product on the int8 digit kernels (what the Affine function class runs)
        yd = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
        assert max_rel_err(yd, y64) <= TIGHT


def _same_non_finite(y, ref, tol):
    """NaN, +Inf and -Inf at the same places, the finite outputs within the product's tolerance."""
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin.any() and (~fin).any()
    assert np.abs(y[fin] - ref[fin]).max() / np.abs(ref[fin]).max() <= tol


def test_affine_digits_special_rows_and_narrow_weights(dev):
    """Rows of x or columns of W holding NaN / Inf: the outputs they reach are the reference's, one by one
    (affine.cpp:87-95: Inf * w = +-Inf by the signs, Inf - Inf = NaN, 0 * Inf = NaN, NaN anywhere = NaN), all others
    untouched; weights that are all zero or powers of two within six binades per column take the three-product form and
    are multiplied exactly."""
    rng = np.random.RandomState(8)
    x = rng.randn(70, 200).astype(np.float32)
    W = (rng.randn(200, 90) * 0.1).astype(np.float32)
    b = rng.randn(90).astype(np.float32)
    clean = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
    x[3, 5] = np.inf
    x[3, 9] = np.inf        # with x[3, 5]: +-Inf or NaN by the signs of W[5, n] and W[9, n]
    x[40, 0] = -np.inf
    x[69, 199] = np.nan
    W[7, 11] = np.nan
    W[8, 12] = np.inf
    x[9, 8] = 0.0           # 0 * Inf
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.affine(x, W, b)
    y = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
    _same_non_finite(y, ref, TIGHT)
    assert np.isnan(y[9, 12]) and np.isnan(y[:, 11]).all() and np.isinf(y[3]).any() and np.isnan(y[3]).any()
    ok = np.ones_like(y, bool)
    ok[[3, 9, 40, 69]] = False
    ok[:, [11, 12]] = False
    assert bits_equal(y[ok], clean[ok])
    for M in (3, 300):      # the contraction spread over the CUs (few rows), and more than one block of marks
        xm = np.tile(x, (5, 1))[:M]
        with np.errstate(invalid="ignore", over="ignore"):
            ref = oracle.affine(xm, W, None)
        _same_non_finite(to_np(kernels.affine_digits(_dev(xm, dev), _dev(W, dev))), ref, TIGHT)
    # powers of two: exponents within 6 of the column's largest, some zeros, both signs
    e = rng.randint(-9, -3, size=(200, 90))
    Wp = (np.where(rng.rand(200, 90) < 0.2, 0.0, 2.0 ** e) * rng.choice([-1.0, 1.0], size=(200, 90))).astype(np.float32)
    xi = np.rint(rng.randn(70, 200) * 64).astype(np.float32) / 64          # exactly representable rows
    yp = to_np(kernels.affine_digits(_dev(xi, dev), _dev(Wp, dev)))
    assert np.array_equal(yp, (xi.astype(np.float64) @ Wp.astype(np.float64)).astype(np.float32))
    Wp[0, 0] = 2.0 ** -20                                                  # one column now spans too many binades
    yw = to_np(kernels.affine_digits(_dev(xi, dev), _dev(Wp, dev)))
    assert max_rel_err(yw, xi.astype(np.float64) @ Wp.astype(np.float64)) <= TIGHT


@pytest.mark.parametrize("M", [1, 2, 3, 8, 13, 16, 17])
@pytest.mark.parametrize("K,N", [(1024, 1024), (1000, 1284), (4099, 516)])
def test_affine_of_a_few_rows(dev, M, K, N):
    """At most 16 rows against real-valued weights of a million elements or more: one fp32 pass over W (slabs of K,
    added in order) instead of the digit operands; against the oracle with and without bias, and NaN / Inf element by
    element as the reference's product gives them."""
    rng = np.random.RandomState(100 * M + K % 7)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.05).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    y = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev)))
    assert max_rel_err(y, oracle.affine(x, W, None)) <= TIGHT
    y = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
    assert max_rel_err(y, oracle.affine(x, W, b)) <= TIGHT
    if M > 2:                       # (rows in between stay finite)
        x[M - 1, K - 1] = np.inf    # the last row of W's last slab
        x[0, 5] = -np.inf
    W[7, 11] = np.nan
    W[K - 1, 12] = np.inf
    if M > 3:
        x[M // 2, K - 1] = 0.0      # 0 * Inf
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.affine(x, W, b)
    y = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev), _dev(b, dev)))
    _same_non_finite(y, ref, TIGHT)


def _fixed_point_rows(rng, M, K, delta=2.0 ** -4, n=8):
    """Rows as FixedPointQuantize (sign, n bits, step delta) leaves them: integers in [-127, 127] times delta."""
    return (rng.randint(-(2 ** (n - 1) - 1), 2 ** (n - 1), size=(M, K)) * delta).astype(np.float32)


def test_digit_operand_of_fixed_point_rows_is_one_digit(dev):
    """Rows whose values are multiples of one power of two and span at most seven bits land in the top digit alone
    under the ordinary row scale (lower digits zero) and are marked as one-digit rows; the scale is the ordinary one."""
    rng = np.random.RandomState(3)
    M, K = 70, 1024
    x = _fixed_point_rows(rng, M, K)
    x[5] = rng.randn(K)                               # a general row
    x[6] = 0.0                                        # all zero: one digit
    x[7] = _fixed_point_rows(rng, 1, K)[0] * 2.0 ** 40   # the unit may be any power of two
    x[8, 3] = 2.0 ** -9                               # one value 32 times finer than the rest: nine bits, not one digit
    x[9] = np.where(rng.rand(K) < 0.5, 32.0, -0.25)   # 128 units of 2^-2: one past the edge
    x[10] = np.where(rng.rand(K) < 0.5, 31.75, -0.25)  # 127 units of 2^-2: the edge
    q, shift, sums, one = unpack_digits(to_np(kernels.split_digits(_dev(x, dev), M, K)), M, K, with_one_digit=True)
    expect = np.ones(M, bool)
    expect[[5, 8, 9]] = False
    assert np.array_equal(one, expect), np.nonzero(one != expect)
    assert np.array_equal(q, np.rint(np.ldexp(x.astype(np.float64), shift[:, None].astype(np.int64))).astype(np.int64))
    assert np.abs(q[one]).max() <= 127 * 65536 and not (q[one] % 65536).any()
    assert shift[0] == 20 and shift[7] == 20 - 40 and shift[10] == 18
    assert np.array_equal(sums[0], q.sum(1))


@pytest.mark.parametrize("M,K,N", [(256, 1024, 640), (1024, 512, 2048), (96, 4096, 300), (2100, 256, 1100)])
def test_one_digit_rows_give_the_bits_of_the_three_digit_product(dev, M, K, N):
    """A tile whose rows are all one-digit rows multiplies the lowest digit only.  The same rows inside tiles that
    also hold a general row (so the tile takes the three-digit path) must give identical bits: both are the exact
    integer sum, converted once.  Also against float64."""
    rng = np.random.RandomState(M + K)
    x = _fixed_point_rows(rng, M, K)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    y1, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev))
    y1 = to_np(y1)
    x3 = x.copy()
    x3[::32] = rng.randn(len(x3[::32]), K)            # one general row in every 32-row block
    y3, _, _ = kernels.binary_weight_affine(_dev(x3, dev), _dev(W, dev), _dev(b, dev))
    y3 = to_np(y3)
    same = np.ones(M, bool)
    same[::32] = False
    assert bits_equal(y1[same], y3[same]), first_mismatch(y1[same], y3[same])
    sgn = np.where(W >= 0, 1.0, -1.0)
    y64 = x.astype(np.float64) @ (sgn * np.abs(W.astype(np.float64)).mean(0)) + b
    assert max_rel_err(y1, y64) <= TIGHT
    ref_y, _, _ = oracle.binary_weight_affine(x[:64], W, b, 1.0)
    assert max_rel_err(y1[:64], ref_y) <= TOL


@pytest.mark.parametrize("M,K,N", [(256, 512, 384), (1024, 1024, 1024), (130, 4096, 200)])
def test_one_digit_rows_times_one_digit_weights(dev, M, K, N):
    """Real-weight product with fixed-point rows of x and power-of-two weights (an INQ layer behind a fixed-point
    quantizer): a single digit product per tile.  Exact, hence equal to the float64 product rounded once, and
    bit-identical to the rows' results inside tiles that take the three-product path."""
    rng = np.random.RandomState(K)
    x = _fixed_point_rows(rng, M, K)
    e = rng.randint(-9, -3, size=(K, N))
    W = (np.where(rng.rand(K, N) < 0.2, 0.0, 2.0 ** e) * rng.choice([-1.0, 1.0], size=(K, N))).astype(np.float32)
    y1 = to_np(kernels.affine_digits(_dev(x, dev), _dev(W, dev)))
    assert np.array_equal(y1, (x.astype(np.float64) @ W.astype(np.float64)).astype(np.float32))
    x3 = x.copy()
    x3[::128] = rng.randn(len(x3[::128]), K)          # one general row in every 128-row tile
    y3 = to_np(kernels.affine_digits(_dev(x3, dev), _dev(W, dev)))
    same = np.ones(M, bool)
    same[::128] = False
    assert bits_equal(y1[same], y3[same])
    Wg = (rng.randn(K, N) * 0.05).astype(np.float32)  # general weights: six products, one-digit rows as three digits
    yg = to_np(kernels.affine_digits(_dev(x, dev), _dev(Wg, dev)))
    assert max_rel_err(yg, x.astype(np.float64) @ Wg.astype(np.float64)) <= TIGHT


@pytest.mark.parametrize("M", [1, 8, 64])
def test_config3_full_width_small_m_vs_oracle(dev, M):
    """Benchmark configuration 3 at K=4096, N=11008 for the M the CPU oracle finishes in seconds."""
    rng = np.random.default_rng(313)
    x = rng.standard_normal((M, 4096), dtype=np.float32)
    W = rng.standard_normal((4096, 11008), dtype=np.float32) * np.float32(0.02)
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, None, 1.0)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev))
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    assert max_rel_err(to_np(y), ref_y) <= TOL
    yc, Wbc = kernels.binary_connect_affine(_dev(x, dev), _dev(W, dev))
    ref_yc, _ = oracle.binary_connect_affine(x, W, None, 1.0)
    assert bits_equal(to_np(Wbc), ref_Wb)
    assert max_rel_err(to_np(yc), ref_yc) <= TOL


@pytest.mark.parametrize("M", [32, 64, 128, 256, 512, 1024, 4096])   # 32, 64: one pass, operands from registers; 128, 256: one walk, signs shared through LDS
def test_config3_full_size_properties(dev, M):
    """At sizes the oracle cannot finish quickly: float64 dot products on sampled rows/columns,
    linearity in x, and consistency between BinaryWeight and BinaryConnect (y_bw = y_bc * alpha)."""
    rng = np.random.default_rng(7)
    K, N = 4096, 11008
    x = rng.standard_normal((M, K), dtype=np.float32)
    W = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    xd, Wd = _dev(x, dev), _dev(W, dev)
    y, Wb, alpha = kernels.binary_weight_affine(xd, Wd)
    yc, _ = kernels.binary_connect_affine(xd, Wd)
    y, yc, alpha = to_np(y), to_np(yc), to_np(alpha)
    assert bits_equal(to_np(Wb), oracle.sign(W, 1.0))
    rows = rng.choice(M, 24, replace=False)
    cols = np.union1d(rng.choice(N, 96, replace=False), [0, 8191, 8192, 8575, 8576, 10999, N - 1])
    sgn = np.sign(W[:, cols]).astype(np.float64)
    ref_c = x[rows].astype(np.float64) @ sgn
    a64 = np.abs(W[:, cols].astype(np.float64)).mean(0)
    assert np.abs(yc[np.ix_(rows, cols)] - ref_c).max() / np.abs(ref_c).max() <= TIGHT
    assert np.abs(y[np.ix_(rows, cols)] - ref_c * a64).max() / np.abs(ref_c * a64).max() <= TIGHT
    np.testing.assert_allclose(y, yc * alpha[None, :], rtol=1e-6, atol=1e-7)
    # linearity: f(2x) == 2 f(x) exactly (power-of-two scaling commutes with every rounding)
    y2, _, _ = kernels.binary_weight_affine(xd * 2, Wd)
    assert bits_equal(to_np(y2), y * 2)


def test_workspace_too_small_is_reported(dev):
    x, W = _data(4, 64, 64)
    ws = torch.empty(256, dtype=torch.uint8, device=dev)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), workspace=ws)
    assert ei.value.code == kernels.ERR_MEMORY


@pytest.mark.parametrize("q0,zeros", [(1.0, False), (0.0, False), (0.0, True)])
@pytest.mark.parametrize("M", [96, 48, 4])   # packed-bit product; one pass on the matrix cores; on the vector ALUs
def test_forward_replays_in_a_hip_graph(dev, M, q0, zeros):
    """BinaryWeightAffine and a FixedPointQuantize in front of it, captured once and replayed with new inputs: the
    entry points allocate nothing, never synchronise and clear their scratch with kernels, so every replay must
    reproduce the eager result bit for bit (eager work and synchronisations run between the replays).  With
    quantize_zero_to = 0 the choice between the matrix-core product and the fp32 product over the signs is made on the
    device (test_binary_weight_affine.py:72 covers that value), with and without exact-zero weights."""
    K, N = 512, 768
    rng = np.random.RandomState(77)
    Wh = (rng.randn(K, N) * 0.02).astype(np.float32)
    if zeros:
        Wh.ravel()[::9] = 0.0
    W = _dev(Wh, dev)
    x = torch.empty(M, K, device=dev)
    xq, y = torch.empty_like(x), torch.empty(M, N, device=dev)
    ws = kernels.binary_affine_workspace(M, K, N, x)

    def step():
        kernels.fixed_point_quantize(x, True, 8, 2.0 ** -4, out=xq)
        return kernels.binary_weight_affine(xq, W, None, q0, workspace=ws, out=y)

    x.copy_(_dev(rng.randn(M, K).astype(np.float32), dev))
    step()                                            # first call outside the capture (one-time kernel attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _, Wb, alpha = step()
    for i in range(4):
        xi = _dev((rng.randn(M, K) * (i + 1)).astype(np.float32), dev)
        x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        got = to_np(y).copy()
        y.zero_()                                     # eager work between the replays
        step()
        torch.cuda.synchronize()
        assert bits_equal(got, to_np(y)), "replay %d differs from the eager result" % i
        ref, _, _ = oracle.binary_weight_affine(oracle.fixed_point_quantize(to_np(xi), True, 8, 2.0 ** -4),
                                                to_np(W), None, q0)
        assert max_rel_err(got, ref) <= TOL


@pytest.mark.parametrize("M", [9, 32, 64, 100])
def test_quantize_zero_to_that_bf16_does_not_hold(dev, M):
    """Sign(0) = 0.3 with exact-zero weights: the one-pass form that feeds bf16 signs to the matrix cores would cut
    0.3 to eight significand bits, so such a value takes the other forms (fp32 arithmetic on the signs)."""
    x, W = _data(M, 256, 260, seed=M)
    W.ravel()[::6] = 0.0
    b = np.random.RandomState(4).randn(260).astype(np.float32)
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, 0.3)
    y, Wb, alpha = kernels.binary_weight_affine(_dev(x, dev), _dev(W, dev), _dev(b, dev), 0.3)
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    y64 = x.astype(np.float64) @ (ref_Wb.astype(np.float64) * np.abs(W.astype(np.float64)).mean(0)) + b
    assert max_rel_err(to_np(y), y64) <= TIGHT and max_rel_err(to_np(y), ref_y) <= TIGHT * 4


def test_product_timer_stamps_its_launches_and_leaves_the_results_alone(dev):
    """The measurement aid of bench.py: armed launches of the bit-weight product carry the runtime's begin / end
    stamps; results are the same bits, launches past the armed number run as usual, reading disarms."""
    x, W = _data(512, 1024, 1024, seed=9)
    xd, Wd = _dev(x, dev), _dev(W, dev)
    y0, _, _ = kernels.binary_weight_affine(xd, Wd)
    kernels.gemm_bits_timer_arm(3)
    ys = [kernels.binary_weight_affine(xd, Wd)[0] for _ in range(5)]
    t = kernels.gemm_bits_timer_read()
    assert t["launches"] == 3
    assert 0.0 < t["min_ms"] <= t["mean_ms"] <= t["max_ms"] < 5.0
    for y in ys:
        assert bits_equal(to_np(y), to_np(y0))
    assert kernels.gemm_bits_timer_read()["launches"] == 0
    with pytest.raises(kernels.KernelError):
        kernels.gemm_bits_timer_arm(0)


@pytest.mark.parametrize("M,K,N,q0", [(100, 1024, 8196, 1.0), (100, 1024, 8196, 0.0), (600, 512, 2052, 1.0)])
def test_one_walk_and_two_walk_forms_and_the_backward_replay_in_a_hip_graph(dev, M, K, N, q0):
    """The forward's one-walk form (some hundred rows, wide outputs; with quantize_zero_to = 0 and exact-zero weights
    its device-side fall-back), the two-walk form, and the backward pass of each, captured once and replayed on new
    inputs: the replay's bits are the eager call's."""
    rng = np.random.RandomState(78)
    Wh = (rng.randn(K, N) * 0.02).astype(np.float32)
    Wh.ravel()[::11] = 0.0
    W = _dev(Wh, dev)
    x, dy = torch.empty(M, K, device=dev), torch.empty(M, N, device=dev)

    def step():
        y, Wb, alpha = kernels.binary_weight_affine(x, W, None, q0)
        dx, dW, db = kernels.binary_affine_backward(dy, x, W, Wb, alpha, q0)
        return y, dx, dW, db

    x.copy_(_dev(rng.randn(M, K).astype(np.float32), dev))
    dy.copy_(_dev(rng.randn(M, N).astype(np.float32), dev))
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for i in range(3):
        x.copy_(_dev((rng.randn(M, K) * (i + 1)).astype(np.float32), dev))
        dy.copy_(_dev(rng.randn(M, N).astype(np.float32), dev))
        graph.replay()
        torch.cuda.synchronize()
        got = [to_np(o).copy() for o in outs]
        eager = step()
        torch.cuda.synchronize()
        for g, e, name in zip(got, eager, ("y", "dx", "dW", "db")):
            assert bits_equal(g, to_np(e)), "replay %d: %s differs from the eager result" % (i, name)
        ref, _, _ = oracle.binary_weight_affine(to_np(x), Wh, None, q0)
        assert max_rel_err(got[0], ref) <= TOL
