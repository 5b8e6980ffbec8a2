"""Grouped convolutions whose groups are small (depthwise, a few channels per group): all groups run in one launch per
kernel, in plain fp32 (conv_direct.hip), forward and backward, for the binary layers and for the real-weight
Convolution; the forward of a single group of very few input channels takes the same kernels.  Against the oracle (convolution.cpp:161-330 restated per sample and group) at the fp32-faithful
tolerance; Wb bit for bit, alpha at the tolerance of a sum in another order; accumulation into the gradients; Sign(0)
that is neither +1 nor -1; windows holding NaN / Inf (the plain fp32 product propagates them as the reference does)."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TIGHT = 5e-6

CASES = [
    # (x shape, w shape, pad, stride, dilation, group)
    ((4, 32, 14, 14), (32, 1, 3, 3), (1, 1), (1, 1), (1, 1), 32),          # depthwise
    ((3, 24, 15, 13), (48, 1, 3, 3), (1, 1), (2, 2), (1, 1), 24),          # channel multiplier 2, stride 2
    ((2, 64, 9, 9), (64, 8, 3, 3), (1, 1), (1, 1), (1, 1), 8),             # eight channels per group
    ((2, 48, 10, 8), (96, 4, 3, 2), (2, 1), (1, 2), (2, 1), 12),           # dilation, uneven stride and padding
    ((3, 20, 40), (20, 1, 5), (2,), (1,), (1,), 20),                        # one spatial dimension
    ((2, 12, 5, 6, 7), (12, 2, 2, 3, 2), (1, 1, 0), (1, 2, 1), (1, 1, 2), 6),  # three
    ((2, 16, 7, 7), (16, 1, 7, 7), (3, 3), (1, 1), (1, 1), 16),            # a kernel as large as the input
    ((16, 8, 12, 12), (8, 1, 5, 5), (2, 2), (1, 1), (1, 1), 8),            # 25 taps; the samples in several runs
    ((40, 16, 6, 6), (32, 4, 3, 3), (1, 1), (1, 1), (1, 1), 4),            # few positions: samples side by side
    # one group of very few input channels under a kernel of many taps (the first layer of an image network): the
    # forward takes the same kernels, eight output channels per thread; the backward the general path
    ((2, 3, 40, 36), (16, 3, 7, 7), (3, 3), (2, 2), (1, 1), 1),
    ((2, 4, 20, 20), (8, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((3, 1, 70, 9), (24, 1, 5, 3), (2, 1), (1, 1), (1, 1), 1),
    ((2, 32, 12, 12), (64, 16, 3, 3), (1, 1), (1, 1), (1, 1), 2),           # sixteen output channels per thread
]


def _dev(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _data(xs, ws, pad, stride, dil, group, seed):
    rng = np.random.RandomState(seed)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)
    y = oracle.convolution(x, W, None, pad, stride, dil, group)
    dy = rng.randn(*y.shape).astype(np.float32)
    return x, W, b, dy


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
def test_forward(dev, xs, ws, pad, stride, dil, group):
    x, W, b, _ = _data(xs, ws, pad, stride, dil, group, 51)
    for bias in (None, b):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, bias, pad, stride, dil, group, 1.0)
        y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), _dev(bias, dev), pad, stride, dil,
                                                         group)
        assert bits_equal(to_np(Wb), ref_Wb)
        assert max_rel_err(to_np(alpha), ref_alpha) <= 2e-6
        assert max_rel_err(to_np(y), ref_y) <= TIGHT
        ref_y, ref_Wb = oracle.binary_connect_convolution(x, W, bias, pad, stride, dil, group, 1.0)
        y, Wb = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), _dev(bias, dev), pad, stride, dil, group)
        assert bits_equal(to_np(Wb), ref_Wb) and max_rel_err(to_np(y), ref_y) <= TIGHT
        Wd = _dev(W, dev)
        I = torch.zeros(ws, dtype=torch.int32, device=dev)
        y = kernels.inq_convolution(_dev(x, dev), Wd, I, Wd.clone(), I.clone(), _dev(bias, dev), pad, stride, dil, group,
                                    4, kernels.INQ_PRODUCT_ONLY)
        assert max_rel_err(to_np(y), oracle.convolution(x, W, bias, pad, stride, dil, group)) <= TIGHT


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
def test_backward(dev, xs, ws, pad, stride, dil, group):
    x, W, _, dy = _data(xs, ws, pad, stride, dil, group, 52)
    d = lambda a: _dev(a, dev)
    rng = np.random.RandomState(6)
    old = [rng.randn(*s).astype(np.float32) for s in (xs, ws, (ws[0],))]
    for alpha in (np.abs(W).reshape(ws[0], -1).mean(1).astype(np.float32), None):
        ref = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0)
        got = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0)
        for g_, r_ in zip(got, ref):
            assert max_rel_err(to_np(g_), r_) <= TIGHT
        ref = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0, dx=old[0], dW=old[1],
                                                 db=old[2])
        got = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0,
                                                  dx=d(old[0]), dW=d(old[1]), db=d(old[2]))
        for g_, r_ in zip(got, ref):
            assert max_rel_err(to_np(g_), r_) <= TIGHT
    ref = oracle.convolution_backward(dy, x, W, pad, stride, dil, group)
    got = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group)
    for g_, r_ in zip(got, ref):
        assert max_rel_err(to_np(g_), r_) <= TIGHT
    only = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group, want=(False, True, False))
    assert only[0] is None and only[2] is None and max_rel_err(to_np(only[1]), ref[1]) <= TIGHT


@pytest.mark.parametrize("q0", [0.0, 0.3, -1.0])
def test_sign_of_zero(dev, q0):
    xs, ws, pad, stride, dil, group = (3, 16, 9, 9), (16, 2, 3, 3), (1, 1), (1, 1), (1, 1), 8
    x, W, b, dy = _data(xs, ws, pad, stride, dil, group, 53)
    W.ravel()[::3] = 0.0
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, pad, stride, dil, group, q0)
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), pad, stride, dil, group, q0)
    assert bits_equal(to_np(Wb), ref_Wb) and max_rel_err(to_np(y), ref_y) <= TIGHT
    ref = oracle.binary_convolution_backward(dy, x, W, ref_alpha, pad, stride, dil, group, q0)
    got = kernels.binary_convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), Wb, alpha, pad, stride, dil,
                                              group, q0)
    for g_, r_ in zip(got, ref):
        assert max_rel_err(to_np(g_), r_) <= TIGHT * 4
    if q0 == -1.0:  # a sign the weights themselves give: the binarised weights need not be passed
        got = kernels.binary_convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), None, alpha, pad, stride,
                                                  dil, group, q0)
        assert max_rel_err(to_np(got[0]), ref[0]) <= TIGHT * 4


def test_non_finite_windows(dev):
    xs, ws, pad, stride, dil, group = (2, 8, 9, 9), (8, 1, 3, 3), (1, 1), (1, 1), (1, 1), 8
    x, W, b, _ = _data(xs, ws, pad, stride, dil, group, 54)
    x[1, 3, 4, 5] = np.inf
    x[0, 0, 0, 0] = np.nan
    x[1, 3, 4, 6] = -np.inf
    with np.errstate(invalid="ignore", over="ignore"):
        ref, _, _ = oracle.binary_weight_convolution(x, W, b, pad, stride, dil, group, 1.0)
    y, _, _ = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), pad, stride, dil, group)
    y = to_np(y)
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref)) and np.isnan(ref).any() and np.isinf(ref).any()
    fin = np.isfinite(ref)
    assert np.abs(y[fin] - ref[fin]).max() <= TIGHT * np.abs(ref[fin]).max()
