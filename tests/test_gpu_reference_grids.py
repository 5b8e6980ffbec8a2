"""The parameter grids of the reference's own function tests (python/test/function/test_binary_weight_affine.py,
test_binary_connect_affine.py, test_binary_*_convolution.py, test_min_max_quantize.py, test_quantize_linear.py,
test_dequantize_linear.py, test_prune.py), run through ``F.*`` under the hip context against the CPU oracle:
the same shapes, base axes (negative ones included), groups, biases and quantize_zero_to values, forward and
backward, and -- as the reference's ``reset`` variants do -- the same function object set up again on inputs of
other shapes."""
import numpy as np
import pytest

import nnabla_amd as nn
import nnabla_amd.functions as F
import oracle
from nnabla_amd.ext_utils import get_extension_context
from util import bits_equal, max_rel_err

pytestmark = pytest.mark.gpu
TIGHT = 5e-6


@pytest.fixture()
def ctx(dev):
    c = get_extension_context('hip', device_id='0')
    with nn.context_scope(c):
        yield c


def _var(a, need_grad=False):
    v = nn.Variable(a.shape, need_grad=need_grad)
    v.d = a
    return v


def _reset(v, a):
    v.reset_shape(a.shape, force=True)
    v.d = a


def _affine_case(rng, x_shape, weight_shape, base_axis, bias):
    x = rng.randn(*x_shape).astype(np.float32)
    W = rng.randn(*weight_shape).astype(np.float32)
    b = rng.randn(*weight_shape[1:]).astype(np.float32) if bias else None
    axis = base_axis if base_axis >= 0 else len(x_shape) + base_axis
    rows = int(np.prod(x_shape[:axis]))
    return x, W, b, axis, rows


# test_binary_weight_affine.py:69-72,98-102 / test_binary_connect_affine.py:67-70,95-99
AFFINE_GRID = [(1, (12, 2, 3), (20, 2, 3)), (2, (4, 4), (5, 4)), (-1, (4, 4), (5, 4)), (-2, (12, 3, 4), (20, 3, 4))]


@pytest.mark.parametrize("base_axis,weight_shape,reset_weight_shape", AFFINE_GRID)
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("quantize_zero_to", [0.0, -1.0, 1.0])
@pytest.mark.parametrize("weight_alpha", [True, False])
def test_binary_affines(ctx, base_axis, weight_shape, reset_weight_shape, bias, quantize_zero_to, weight_alpha):
    rng = np.random.RandomState(313)
    xv, wv, wbv, av, bv = (nn.Variable((1,)) for _ in range(5))
    xv.need_grad = wv.need_grad = bv.need_grad = True
    y = None
    for x_shape, w_shape in (((2, 3, 4), weight_shape), ((3, 4, 5), reset_weight_shape)):
        x, W, b, axis, rows = _affine_case(rng, x_shape, w_shape, base_axis, bias)
        W.ravel()[::5] = 0.0                                   # Sign(0) = quantize_zero_to is in play
        n = int(np.prod(w_shape[1:]))
        _reset(xv, x), _reset(wv, W), _reset(wbv, np.zeros_like(W)), _reset(av, np.zeros(n, np.float32))
        if bias:
            _reset(bv, b)
        if y is None:
            if weight_alpha:
                y = F.binary_weight_affine(xv, wv, wbv, av, bv if bias else None, base_axis, quantize_zero_to)
            else:
                y = F.binary_connect_affine(xv, wv, wbv, bv if bias else None, base_axis, quantize_zero_to)
        y.forward()
        x2, W2 = x.reshape(rows, -1), W.reshape(W.shape[0], -1)
        b2 = None if b is None else b.ravel()
        if weight_alpha:
            ref_y, ref_wb, ref_alpha = oracle.binary_weight_affine(x2, W2, b2, quantize_zero_to)
            np.testing.assert_allclose(av.d, ref_alpha, rtol=2e-6)
        else:
            ref_y, ref_wb = oracle.binary_connect_affine(x2, W2, b2, quantize_zero_to)
            ref_alpha = None
        assert y.shape == tuple(x_shape[:axis]) + tuple(w_shape[1:])
        assert bits_equal(wbv.d.reshape(W2.shape), ref_wb)
        assert max_rel_err(y.d.reshape(rows, n), ref_y) <= TIGHT
        dy = rng.randn(*y.shape).astype(np.float32)
        for v in (xv, wv, bv):
            v.grad.zero()
        y.backward(dy)
        rdx, rdw, rdb = oracle.binary_affine_backward(dy.reshape(rows, n), x2, W2, ref_alpha, quantize_zero_to)
        assert max_rel_err(xv.g.reshape(rows, -1), rdx) <= TIGHT
        assert max_rel_err(wv.g.reshape(W2.shape), rdw) <= TIGHT
        if bias:
            assert max_rel_err(bv.g.ravel(), rdb) <= TIGHT


# test_binary_weight_convolution.py:74-78,103-107 / test_binary_connect_convolution.py:74-79,104-109
@pytest.mark.parametrize("group", [1, 2])
@pytest.mark.parametrize("base_axis", [1, -3])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("quantize_zero_to", [0.0, -1.0, 1.0])
@pytest.mark.parametrize("weight_alpha", [True, False])
def test_binary_convolutions(ctx, group, base_axis, with_bias, quantize_zero_to, weight_alpha):
    rng = np.random.RandomState(313)
    pad, stride, dilation = (3, 0), (1, 2), (2, 1)
    xv, wv, wbv, av, bv = (nn.Variable((1,)) for _ in range(5))
    xv.need_grad = wv.need_grad = bv.need_grad = True
    y = None
    for inshape, kernel, outmaps in (((2, 2, 10, 10), (3, 2), 4), ((3, 2, 12, 12), (2, 2), 6)):
        x = rng.randn(*inshape).astype(np.float32)
        W = rng.randn(outmaps, inshape[1] // group, *kernel).astype(np.float32)
        W.ravel()[::7] = 0.0
        b = rng.randn(outmaps).astype(np.float32) if with_bias else None
        _reset(xv, x), _reset(wv, W), _reset(wbv, np.zeros_like(W)), _reset(av, np.zeros(outmaps, np.float32))
        if with_bias:
            _reset(bv, b)
        if y is None:
            if weight_alpha:
                y = F.binary_weight_convolution(xv, wv, wbv, av, bv if with_bias else None, base_axis, pad, stride,
                                                dilation, group, quantize_zero_to)
            else:
                y = F.binary_connect_convolution(xv, wv, wbv, bv if with_bias else None, base_axis, pad, stride,
                                                 dilation, group, quantize_zero_to)
        y.forward()
        if weight_alpha:
            ref_y, ref_wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, pad, stride, dilation, group,
                                                                        quantize_zero_to)
            np.testing.assert_allclose(av.d, ref_alpha, rtol=2e-6)
        else:
            ref_y, ref_wb = oracle.binary_connect_convolution(x, W, b, pad, stride, dilation, group, quantize_zero_to)
            ref_alpha = None
        assert y.shape == ref_y.shape and bits_equal(wbv.d, ref_wb)
        assert max_rel_err(y.d, ref_y) <= TIGHT
        dy = rng.randn(*y.shape).astype(np.float32)
        for v in (xv, wv, bv):
            v.grad.zero()
        y.backward(dy)
        rdx, rdw, rdb = oracle.binary_convolution_backward(dy, x, W, ref_alpha, pad, stride, dilation, group,
                                                           quantize_zero_to)
        assert max_rel_err(xv.g, rdx) <= TIGHT * 4 and max_rel_err(wv.g, rdw) <= TIGHT
        if with_bias:
            assert max_rel_err(bv.g, rdb) <= TIGHT


# test_min_max_quantize.py:199-207: the same function set up again for per-output-channel weights
@pytest.mark.parametrize("decay", [0.999, 0.9])
@pytest.mark.parametrize("ste_fine_grained", [True, False])
def test_min_max_quantize_set_up_again(ctx, decay, ste_fine_grained):
    rng = np.random.RandomState(313)
    xv, lo, hi, ql, qh = (nn.Variable((1,)) for _ in range(5))
    xv.need_grad = True
    y = None
    for x_shape, q_shape in (((4, 8, 16, 16), (1, 8, 1, 1)), ((16, 8, 3, 3), (16, 1, 1, 1))):
        x = rng.randn(*x_shape).astype(np.float32)
        qmn, qmx = np.full(q_shape, -0.5, np.float32), np.full(q_shape, 0.5, np.float32)
        lmn, lmx = np.zeros(q_shape, np.float32), np.full(q_shape, 255, np.float32)
        _reset(xv, x), _reset(lo, qmn), _reset(hi, qmx), _reset(ql, lmn), _reset(qh, lmx)
        if y is None:
            y = F.min_max_quantize(xv, lo, hi, ql, qh, decay, False, False, ste_fine_grained)
        y.forward()
        ref_y, rmn, rmx, rscale = oracle.min_max_quantize(x, qmn, qmx, lmn, lmx, decay, False, False, 0.01)
        assert bits_equal(y.d, ref_y) and bits_equal(lo.d, rmn) and bits_equal(hi.d, rmx)
        dy = rng.randn(*x_shape).astype(np.float32)
        xv.grad.zero()
        y.backward(dy)
        rdx, _, _ = oracle.min_max_quantize_backward(dy, x, rmn, rmx, lmn, lmx, rscale, ste_fine_grained, False, False)
        assert np.array_equal(xv.g, rdx)      # (accumulated onto a zeroed gradient: -0 arrives as +0)


# test_quantize_linear.py:49-55,104-110 / test_dequantize_linear.py:38,79
@pytest.mark.parametrize("shapes", [[((2, 4, 8, 8), (1, 1, 1, 1)), ((2, 4, 8, 8), (1, 4, 1, 1))],
                                    [((2, 4, 8, 8), (1, 4, 1, 1)), ((2, 8, 8, 4), (1, 1, 1, 4))]])
@pytest.mark.parametrize("round_mode", ["HALF_AWAY_FROM_ZERO", "HALF_TO_EVEN"])
@pytest.mark.parametrize("narrow_range", [False, True])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_quantize_and_dequantize_linear(ctx, shapes, round_mode, narrow_range, dtype):
    rng = np.random.RandomState(313)
    code = {np.int8: 1, np.uint8: 2}[dtype]
    xv, sv, zv = (nn.Variable((1,)) for _ in range(3))
    y = z = None
    for x_shape, s_shape in shapes:
        x = (rng.randn(*x_shape) * 40).astype(np.float32)
        scale = (0.1 + rng.rand(*s_shape)).astype(np.float32)
        zp = np.round(rng.randn(*s_shape) * 3).astype(np.float32)
        _reset(xv, x), _reset(sv, scale), _reset(zv, zp.copy())
        if y is None:
            y = F.quantize_linear(xv, sv, zv, round_mode, narrow_range, code)
            z = F.dequantize_linear(y, sv, zv)
        z.forward()
        ref_y, ref_zp = oracle.quantize_linear(x, scale, zp, round_mode, narrow_range, code)
        assert bits_equal(y.d, ref_y)
        assert bits_equal(z.d, oracle.dequantize_linear(ref_y, scale, ref_zp))


# test_prune.py:45
@pytest.mark.parametrize("rate", [0.0, 0.85, 0.9, 0.95, 1.0])
def test_prune(ctx, rate):
    rng = np.random.RandomState(313)
    for shape in ((2, 3, 4), (5, 7, 11)):
        x = rng.randn(*shape).astype(np.float32)
        y = F.prune(_var(x), rate)
        y.forward()
        assert bits_equal(y.d, oracle.prune(x, rate))


# test_inq_affine.py:119-122 (forward / backward from random indicators) and :150-155 (recomputation)
@pytest.mark.parametrize("base_axis,weight_shape,num_bits",
                         [(1, (12, 2, 3), 2), (2, (4, 4), 4), (-2, (12, 2, 3), 2), (-1, (4, 4), 4)])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("inq_iterations", [(10, 20), (0,), (0, 10)])
def test_inq_affine(ctx, base_axis, weight_shape, num_bits, bias, inq_iterations):
    rng = np.random.RandomState(313)
    x, W, b, axis, rows = _affine_case(rng, (2, 3, 4), weight_shape, base_axis, bias)
    I = rng.randint(2, size=weight_shape).astype(np.int32)
    n = int(np.prod(weight_shape[1:]))
    xv, wv = _var(x, True), _var(W, True)
    iv = nn.Variable(weight_shape)
    iv.set_data(I, np.int32)
    bv = _var(b, True) if bias else None
    y = F.inq_affine(xv, wv, iv, bv, base_axis, num_bits, inq_iterations, 'largest_abs', 313)
    y.forward()
    inq = oracle.Inq(W.size, num_bits, inq_iterations, 'largest_abs', 313)
    Wc, Ic = W.reshape(W.shape[0], -1).copy(), I.reshape(W.shape[0], -1).copy()
    ref_y = inq.affine(x.reshape(rows, -1), Wc, Ic, None if b is None else b.ravel())
    assert np.array_equal(iv.d.astype(np.int32).reshape(Ic.shape), Ic)
    assert bits_equal(wv.d.reshape(Wc.shape), Wc)
    assert max_rel_err(y.d.reshape(rows, n), ref_y) <= TIGHT
    dy = rng.randn(*y.shape).astype(np.float32)
    y.backward(dy)
    rdx, rdw, rdb = oracle.affine_backward(dy.reshape(rows, n), x.reshape(rows, -1), Wc)
    assert max_rel_err(xv.g.reshape(rows, -1), rdx) <= TIGHT and max_rel_err(wv.g.reshape(Wc.shape), rdw) <= TIGHT
    if bias:
        assert max_rel_err(bv.g.ravel(), rdb) <= TIGHT


@pytest.mark.parametrize("base_axis,weight_shape,num_bits", [(1, (12, 2, 3), 2), (2, (4, 4), 4)])
@pytest.mark.parametrize("selection_algorithm", ["largest_abs", "random"])
@pytest.mark.parametrize("func_seed", [-1, 412])
def test_inq_affine_recomputation(ctx, base_axis, weight_shape, num_bits, selection_algorithm, func_seed):
    """The output recomputed after a forward (weights, indicators and counter left as they are) equals the forward's
    (nbla_test_utils.recomputation_test), also at a selection step and with the generator seeded by the clock."""
    rng = np.random.RandomState(313)
    x, W, _, _, _ = _affine_case(rng, (2, 3, 4), weight_shape, base_axis, False)
    iv = nn.Variable(weight_shape)
    iv.set_data(rng.randint(2, size=weight_shape), np.int32)
    wv = _var(W)
    y = F.inq_affine(_var(x), wv, iv, None, base_axis, num_bits, (1,), selection_algorithm, func_seed)
    for _ in range(3):                     # the second forward is the selection step
        y.forward()
        out, w_after, i_after = y.d.copy(), wv.d.copy(), iv.d.copy()
        y.parent.recompute()
        assert bits_equal(y.d, out) and bits_equal(wv.d, w_after) and np.array_equal(iv.d, i_after)


# test_inq_convolution.py:123-128
@pytest.mark.parametrize("group", [1, 2])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("base_axis", [1, -3])
@pytest.mark.parametrize("inq_iterations", [(10, 20), (0,), (0, 10)])
def test_inq_convolution(ctx, group, with_bias, base_axis, inq_iterations):
    rng = np.random.RandomState(313)
    inshape, kernel, outmaps, pad, stride, dilation, num_bits = (2, 2, 10, 10), (3, 2), 4, (3, 0), (1, 2), (2, 1), 3
    x = rng.randn(*inshape).astype(np.float32)
    W = rng.randn(outmaps, inshape[1] // group, *kernel).astype(np.float32)
    I = rng.randint(2, size=W.shape).astype(np.int32)
    b = rng.randn(outmaps).astype(np.float32) if with_bias else None
    xv, wv = _var(x, True), _var(W, True)
    iv = nn.Variable(W.shape)
    iv.set_data(I, np.int32)
    bv = _var(b, True) if with_bias else None
    y = F.inq_convolution(xv, wv, iv, bv, base_axis, pad, stride, dilation, group, num_bits, inq_iterations,
                          'largest_abs', 313)
    y.forward()
    inq = oracle.Inq(W.size, num_bits, inq_iterations, 'largest_abs', 313)
    Wc, Ic = W.copy(), I.copy()
    ref_y = inq.convolution(x, Wc, Ic, b, pad, stride, dilation, group)
    assert np.array_equal(iv.d.astype(np.int32), Ic) and bits_equal(wv.d, Wc)
    assert y.shape == ref_y.shape and max_rel_err(y.d, ref_y) <= TIGHT
    dy = rng.randn(*y.shape).astype(np.float32)
    y.backward(dy)
    rdx, rdw, rdb = oracle.convolution_backward(dy, x, Wc, pad, stride, dilation, group)
    assert max_rel_err(xv.g, rdx) <= TIGHT * 4 and max_rel_err(wv.g, rdw) <= TIGHT
    if with_bias:
        assert max_rel_err(bv.g, rdb) <= TIGHT


# test_fixed_point_quantize.py:67-71 and test_pow2_quantize.py:75-80
@pytest.mark.parametrize("sign", [False, True])
@pytest.mark.parametrize("n", [3, 8])
@pytest.mark.parametrize("delta", [2 ** -7, 0.005])
@pytest.mark.parametrize("quantize", [False, True])
@pytest.mark.parametrize("ste_fine_grained", [False, True])
def test_fixed_point_quantize(ctx, sign, n, delta, quantize, ste_fine_grained):
    rng = np.random.RandomState(313)
    x = rng.randn(2, 3, 4).astype(np.float32)
    xv = _var(x, True)
    with nn.auto_forward(False):
        y = F.fixed_point_quantize(xv, sign, n, delta, quantize, ste_fine_grained)
    if not quantize:
        assert y is xv                      # the reference returns its input (functions.py: `if not quantize`)
        return
    y.forward()
    assert bits_equal(y.d, oracle.fixed_point_quantize(x, sign, n, delta))
    dy = rng.randn(2, 3, 4).astype(np.float32)
    y.backward(dy)
    assert np.array_equal(xv.g, oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, ste_fine_grained))


@pytest.mark.parametrize("sign", [False, True])
@pytest.mark.parametrize("with_zero", [False, True])
@pytest.mark.parametrize("n", [3, 5])
@pytest.mark.parametrize("m", [0, 1])
@pytest.mark.parametrize("quantize", [False, True])
@pytest.mark.parametrize("ste_fine_grained", [False, True])
def test_pow2_quantize(ctx, sign, with_zero, n, m, quantize, ste_fine_grained):
    rng = np.random.RandomState(313)
    x = rng.randn(2, 3, 4).astype(np.float32)
    xv = _var(x, True)
    y = F.pow2_quantize(xv, sign, with_zero, n, m, quantize, ste_fine_grained)
    if not quantize:
        assert y is xv
        return
    y.forward()
    assert bits_equal(y.d, oracle.pow2_quantize(x, sign, with_zero, n, m))
    dy = rng.randn(2, 3, 4).astype(np.float32)
    y.backward(dy)
    assert np.array_equal(xv.g, oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, ste_fine_grained))


# test_min_max_quantize.py:114-126
@pytest.mark.parametrize("x_shape,q_shape", [((4, 8, 16, 16), (1, 1, 1, 1)), ((4, 8, 16, 16), (1, 8, 1, 1)),
                                             ((16, 8, 3, 3), (16, 1, 1, 1))])
@pytest.mark.parametrize("decay", [0.999, 0.9])
@pytest.mark.parametrize("x_min_max", [True, False])
@pytest.mark.parametrize("ema", [True, False])
@pytest.mark.parametrize("ste_fine_grained", [True, False])
def test_min_max_quantize(ctx, x_shape, q_shape, decay, x_min_max, ema, ste_fine_grained):
    rng = np.random.RandomState(313)
    x = rng.randn(*x_shape).astype(np.float32)
    qmn, qmx = np.full(q_shape, -0.5, np.float32), np.full(q_shape, 0.5, np.float32)
    lmn, lmx = np.zeros(q_shape, np.float32), np.full(q_shape, 255, np.float32)
    xv, lo, hi = _var(x, True), _var(qmn), _var(qmx)
    y = F.min_max_quantize(xv, lo, hi, _var(lmn), _var(lmx), decay, x_min_max, ema, ste_fine_grained, 0.01)
    y.forward()
    ref_y, rmn, rmx, rscale = oracle.min_max_quantize(x, qmn, qmx, lmn, lmx, decay, x_min_max, ema, 0.01)
    assert bits_equal(y.d, ref_y) and bits_equal(lo.d, rmn) and bits_equal(hi.d, rmx)
    dy = rng.randn(*x_shape).astype(np.float32)
    y.backward(dy)
    rdx, _, _ = oracle.min_max_quantize_backward(dy, x, rmn, rmx, lmn, lmx, rscale, ste_fine_grained, x_min_max, ema)
    assert np.array_equal(xv.g, rdx)
