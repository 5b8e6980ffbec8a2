"""Pins of the oracle's backward restatements (CPU only): closed forms from the reference text
(fixed_point_quantize.cpp:69-127, pow2_quantize.cpp:84-156, min_max_quantize.cpp:225-350) written independently in
numpy, the accumulate/overwrite rules, and the cases the straight-through estimators special-case."""
import numpy as np
import pytest

import oracle


def _rand(shape, seed, scale=1.0):
    return (np.random.RandomState(seed).randn(*shape) * scale).astype(np.float32)


@pytest.mark.parametrize("sign,n,delta", [(True, 8, 2.0 ** -4), (False, 4, 0.1), (True, 3, 0.25)])
def test_fixed_point_backward_mask(sign, n, delta):
    x = _rand((5, 37), 1, 6.0)
    dy = _rand((5, 37), 2)
    nn = n - 1 if sign else n
    hi = np.float32((2 ** nn - 1) * delta)
    lo = np.float32(-hi) if sign else np.float32(0)
    x.ravel()[:4] = [hi, lo, np.nextafter(hi, np.float32(np.inf)), np.nextafter(lo, np.float32(-np.inf))]
    inside = (x <= hi) & (x >= lo)
    assert np.array_equal(oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, True), np.where(inside, dy, 0))
    old = _rand((5, 37), 3)
    # outside the range an accumulated gradient is left untouched; inside dy is added
    assert np.array_equal(oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, True, dx=old),
                          np.where(inside, old + dy, old))
    assert np.array_equal(oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, False), dy)
    assert np.array_equal(oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, False, dx=old), old + dy)


@pytest.mark.parametrize("sign,with_zero,n,m", [(True, True, 4, 1), (False, True, 4, 0), (True, False, 3, -2),
                                                (False, False, 2, 3)])
def test_pow2_backward_mask(sign, with_zero, n, m):
    x = _rand((4, 50), 5, 2.0 ** m)
    dy = _rand((4, 50), 6)
    x.ravel()[:6] = [0.0, -0.0, 2.0 ** m, 2.0 ** m * 1.4, 2.0 ** m * 1.5, -(2.0 ** m) * 3]
    # 2^round(log2|x|) > 2^m  <=>  round(log2|x|) > m; away from the sqrt(2) windows float64 decides it
    with np.errstate(divide="ignore"):
        r = np.round(np.log2(np.abs(x.astype(np.float64))))
    c = np.where(r > m, 0.0, 1.0)
    if not sign:
        c = np.where(x < 0, 0.0, c)
    got = oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, True)
    assert np.array_equal(got, (c * dy).astype(np.float32))
    old = _rand((4, 50), 7)
    got = oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, True, dx=old)
    assert np.array_equal(got, old + (c * dy).astype(np.float32))
    assert np.array_equal(oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, False), dy)


def test_pow2_backward_product_keeps_ieee_cases():
    """dx = c * dy is a product: a zero factor turns an infinite dy into NaN and keeps the sign of zero."""
    x = np.array([100.0, 100.0, -100.0], np.float32)
    dy = np.array([np.inf, -3.0, 2.0], np.float32)
    got = oracle.pow2_quantize_backward(dy, x, True, True, 4, 1, True)
    assert np.isnan(got[0]) and got[1] == 0 and np.signbit(got[1]) and got[2] == 0 and not np.signbit(got[2])


@pytest.mark.parametrize("qshape", [(1, 1, 1, 1), (1, 6, 1, 1), (4, 1, 1, 1)])
@pytest.mark.parametrize("fine", [True, False])
def test_min_max_backward(qshape, fine):
    x = _rand((4, 6, 5, 3), 11, 3.0)
    dy = _rand((4, 6, 5, 3), 12)
    qr_min = np.full(qshape, -2.0, np.float32) + _rand(qshape, 13, 0.1)
    qr_max = np.full(qshape, 2.5, np.float32) + _rand(qshape, 14, 0.1)
    ql_min = np.zeros(qshape, np.float32)
    ql_max = np.full(qshape, 255.0, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, 0.999, False, False, 0.01)
    # nudged range in float64 (exact enough away from ties of the zero point)
    zp = np.clip(np.round(ql_min - qmn.astype(np.float64) / scale), ql_min, ql_max)
    m_n = ((ql_min - zp) * scale).astype(np.float32)
    M_n = ((ql_max - zp) * scale).astype(np.float32)
    dx, gmin, gmax = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, fine, False, False)
    inside = (x >= m_n) & (x <= M_n)
    assert np.array_equal(dx, np.where(inside, dy, 0).astype(np.float32) if fine else dy)
    axes = tuple(i for i in range(4) if qshape[i] == 1)
    ref_min = np.where(x < m_n, dy, 0).astype(np.float64).sum(axis=axes, keepdims=True)
    ref_max = np.where(x > M_n, dy, 0).astype(np.float64).sum(axis=axes, keepdims=True)
    np.testing.assert_allclose(gmin, ref_min, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gmax, ref_max, rtol=1e-5, atol=1e-5)
    # accumulation onto given gradients
    odx, omin, omax = _rand(x.shape, 15), _rand(qshape, 16), _rand(qshape, 17)
    dx2, gmin2, gmax2 = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, fine, False, False,
                                                         dx=odx, g_qr_min=omin, g_qr_max=omax)
    assert np.array_equal(dx2, dx + odx)
    np.testing.assert_allclose(gmin2, omin + gmin, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gmax2, omax + gmax, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("x_min_max,ema", [(True, False), (False, True), (True, True)])
def test_min_max_backward_no_range_gradient_with_statistics(x_min_max, ema):
    """min_max_quantize.cpp:294-295: with x_min_max or ema the range parameters receive no gradient."""
    x = _rand((2, 3, 4, 4), 21)
    dy = _rand((2, 3, 4, 4), 22)
    q = lambda v: np.full((1, 1, 1, 1), v, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, q(-1), q(1), q(0), q(255), 0.999, x_min_max, ema, 0.01)
    sentinel = q(7.0)
    dx, gmin, gmax = oracle.min_max_quantize_backward(dy, x, qmn, qmx, q(0), q(255), scale, True, x_min_max, ema,
                                                      g_qr_min=sentinel, g_qr_max=sentinel)
    assert gmin == 7.0 and gmax == 7.0 and dx.shape == x.shape


@pytest.mark.parametrize("M,K,N", [(3, 5, 4), (17, 33, 29)])
def test_affine_backward_against_float64(M, K, N):
    """affine.cpp:98-140: dx = dy.W^T, dW = x^T.dy, db = column sums; accumulation adds to what was there."""
    rng = np.random.RandomState(41)
    x, W, dy = rng.randn(M, K).astype(np.float32), rng.randn(K, N).astype(np.float32), rng.randn(M, N).astype(np.float32)
    dx, dW, db = oracle.affine_backward(dy, x, W)
    np.testing.assert_allclose(dx, dy.astype(np.float64) @ W.astype(np.float64).T, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dW, x.astype(np.float64).T @ dy.astype(np.float64), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, dy.astype(np.float64).sum(0), rtol=1e-5, atol=1e-5)
    o = [rng.randn(*s).astype(np.float32) for s in ((M, K), (K, N), (N,))]
    dx2, dW2, db2 = oracle.affine_backward(dy, x, W, dx=o[0], dW=o[1], db=o[2])
    assert np.array_equal(dx2, o[0] + dx) and np.array_equal(dW2, o[1] + dW) and np.array_equal(db2, o[2] + db)
    only = oracle.affine_backward(dy, x, W, want=(False, False, True))
    assert only[0] is None and only[1] is None and np.array_equal(only[2], db)


@pytest.mark.parametrize("q0", [1.0, 0.0, -1.0])
def test_binary_affine_backward_uses_scaled_signs_and_full_ste(q0):
    """binary_weight_affine.cpp:124-146: the input gradient sees Sign(W) * alpha, the weight gradient is x^T.dy
    untouched by the binarisation (it does not depend on W at all)."""
    rng = np.random.RandomState(42)
    M, K, N = 6, 9, 7
    x, W, dy = rng.randn(M, K).astype(np.float32), rng.randn(K, N).astype(np.float32), rng.randn(M, N).astype(np.float32)
    W.ravel()[::4] = 0.0
    alpha = np.abs(W).mean(0).astype(np.float32)
    ws = np.where(W > 0, 1.0, np.where(W < 0, -1.0, q0)).astype(np.float32) * alpha
    dx, dW, db = oracle.binary_affine_backward(dy, x, W, alpha, q0)
    rdx, rdW, rdb = oracle.affine_backward(dy, x, ws)
    assert np.array_equal(dx, rdx) and np.array_equal(dW, rdW) and np.array_equal(db, rdb)
    dW_other = oracle.binary_affine_backward(dy, x, -3.0 * W + 1.0, alpha, q0)[1]
    assert np.array_equal(dW_other, dW)
    # BinaryConnect: no alpha
    dxc = oracle.binary_affine_backward(dy, x, W, None, q0)[0]
    assert np.array_equal(dxc, oracle.affine_backward(dy, x, np.where(W > 0, 1.0, np.where(W < 0, -1.0, q0)))[0])


CONV_CASES = [
    # (x shape, W shape, pad, stride, dilation, group)
    ((2, 4, 7, 6), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((3, 4, 9, 8), (4, 2, 3, 2), (2, 0), (2, 1), (1, 2), 2),
    ((2, 6, 11), (3, 2, 4), (1,), (3,), (2,), 3),
    ((1, 2, 5, 6, 4), (4, 2, 2, 3, 1), (1, 1, 0), (1, 2, 1), (1, 1, 1), 1),
]


def _torch_conv_grads(x, W, b, dy, pad, stride, dilation, group):
    """Gradients by torch's CPU autograd in float64: an independent library routine for the same operator."""
    import torch
    import torch.nn.functional as tf
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(W, dtype=torch.float64, requires_grad=True)
    tb = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    conv = {1: tf.conv1d, 2: tf.conv2d, 3: tf.conv3d}[W.ndim - 2]
    y = conv(tx, tw, tb, stride=stride, padding=pad, dilation=dilation, groups=group)
    y.backward(torch.tensor(dy, dtype=torch.float64))
    return tx.grad.numpy(), tw.grad.numpy(), tb.grad.numpy()


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CONV_CASES)
def test_convolution_backward_against_autograd(xs, ws, pad, stride, dil, group):
    x, W, b = _rand(xs, 11), _rand(ws, 12, 0.3), _rand((ws[0],), 13)
    y = oracle.convolution(x, W, b, pad, stride, dil, group)
    dy = _rand(y.shape, 14)
    rdx, rdw, rdb = _torch_conv_grads(x, W, b, dy, pad, stride, dil, group)
    dx, dw, db = oracle.convolution_backward(dy, x, W, pad, stride, dil, group)
    np.testing.assert_allclose(dx, rdx, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dw, rdw, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(db, rdb, rtol=2e-5, atol=2e-5)
    # accumulation onto existing gradients, and outputs that are not asked for stay untouched
    ox, ow, ob = _rand(xs, 15), _rand(ws, 16), _rand((ws[0],), 17)
    ax, aw, ab = oracle.convolution_backward(dy, x, W, pad, stride, dil, group, dx=ox, dW=ow, db=ob)
    np.testing.assert_allclose(ax, ox + rdx, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(aw, ow + rdw, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(ab, ob + rdb, rtol=2e-5, atol=2e-5)
    only_w = oracle.convolution_backward(dy, x, W, pad, stride, dil, group, want=(False, True, False))
    assert only_w[0] is None and only_w[2] is None and np.array_equal(only_w[1], dw)


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CONV_CASES[:3])
@pytest.mark.parametrize("weight_scaled", [True, False])
def test_binary_convolution_backward_is_convolution_backward_of_sign_weights(xs, ws, pad, stride, dil, group,
                                                                             weight_scaled):
    """dx and db are those of a convolution with Sign(W) (* alpha per output channel); the weight gradient is the
    one w.r.t. those weights handed straight through onto W (no factor alpha, no mask)."""
    x, W = _rand(xs, 21), _rand(ws, 22, 0.3)
    W.ravel()[:3] = [0.0, -0.0, 1e-30]
    q0 = -1.0
    if weight_scaled:
        _, Wb, alpha = oracle.binary_weight_convolution(x, W, None, pad, stride, dil, group, q0)
        Ws = Wb * alpha.reshape((-1,) + (1,) * (W.ndim - 1))
    else:
        _, Wb = oracle.binary_connect_convolution(x, W, None, pad, stride, dil, group, q0)
        alpha, Ws = None, Wb
    assert Wb.ravel()[0] == -1.0 and Wb.ravel()[1] == -1.0 and Wb.ravel()[2] == 1.0
    y = oracle.convolution(x, Ws, None, pad, stride, dil, group)
    dy = _rand(y.shape, 23)
    rdx, rdw, rdb = _torch_conv_grads(x, Ws, np.zeros(ws[0], np.float32), dy, pad, stride, dil, group)
    dx, dw, db = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, q0)
    np.testing.assert_allclose(dx, rdx, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dw, rdw, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(db, rdb, rtol=2e-5, atol=2e-5)
    ow = _rand(ws, 24)
    _, aw, _ = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, q0, dW=ow)
    np.testing.assert_allclose(aw, ow + rdw, rtol=2e-5, atol=2e-5)
