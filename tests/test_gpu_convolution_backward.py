"""GPU parity of the convolution backward passes (BinaryWeightConvolution, BinaryConnectConvolution and the
real-weight Convolution inside INQConvolution) against the CPU oracle at the north-star tolerance (1e-4 of the
largest magnitude) and at the fp32-faithful one, plus accumulation and not-propagated outputs."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import max_rel_err, to_np

pytestmark = pytest.mark.gpu
TOL, TIGHT = 1e-4, 5e-6

CASES = [
    # (x shape, w shape, pad, stride, dilation, group)
    ((2, 4, 7, 7), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 4, 7, 7), (6, 2, 3, 3), (1, 0), (2, 1), (1, 2), 2),
    ((1, 3, 9, 8), (5, 3, 2, 3), (0, 2), (1, 2), (2, 1), 1),
    ((3, 2, 10), (4, 2, 3), (1,), (2,), (1,), 1),
    ((2, 2, 4, 5, 6), (3, 2, 2, 3, 2), (1, 0, 1), (1, 2, 1), (1, 1, 2), 1),
    ((2, 6, 5, 5), (6, 1, 3, 3), (1, 1), (1, 1), (1, 1), 6),
    ((4, 8, 16, 16), (16, 8, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((3, 64, 14, 14), (96, 32, 3, 3), (1, 1), (1, 1), (1, 1), 2),
    # unit stride and 24 output channels per group or more: the input gradient of the binary layers runs as a binary
    # convolution of dy (channels' roles exchanged, taps flipped, padding (k - 1) dil - pad).  32 channels exactly;
    # dilation with no padding; one and three spatial dimensions; a padding larger than the kernel (the flipped
    # convolution would need a negative one: the unfolded form runs)
    ((2, 8, 9, 9), (32, 8, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 8, 10, 9), (40, 8, 3, 2), (0, 1), (1, 1), (2, 1), 1),
    ((3, 4, 30), (32, 4, 5), (2,), (1,), (1,), 1),
    ((1, 3, 4, 5, 6), (32, 3, 2, 3, 2), (1, 0, 1), (1, 1, 1), (1, 1, 2), 1),
    ((2, 4, 6, 6), (32, 4, 2, 2), (3, 3), (1, 1), (1, 1), 1),
]


def _dev(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _data(xs, ws, pad, stride, dil, group, seed):
    rng = np.random.RandomState(seed)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    y = oracle.convolution(x, W, None, pad, stride, dil, group)
    dy = rng.randn(*y.shape).astype(np.float32)
    return x, W, dy


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
@pytest.mark.parametrize("with_alpha", [True, False])
def test_binary_convolution_backward(dev, xs, ws, pad, stride, dil, group, with_alpha):
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 41)
    alpha = np.abs(W).reshape(ws[0], -1).mean(1).astype(np.float32) if with_alpha else None
    rdx, rdw, rdb = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0)
    gdx, gdw, gdb = kernels.binary_convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), None,
                                                        _dev(alpha, dev), pad, stride, dil, group, 1.0)
    assert tuple(gdx.shape) == x.shape and tuple(gdw.shape) == W.shape
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
def test_convolution_backward_real_weights(dev, xs, ws, pad, stride, dil, group):
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 42)
    rdx, rdw, rdb = oracle.convolution_backward(dy, x, W, pad, stride, dil, group)
    gdx, gdw, gdb = kernels.convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), pad, stride, dil, group)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT


@pytest.mark.parametrize("q0", [0.0, 0.5, -1.0])
def test_binary_convolution_backward_zero_weights(dev, q0):
    """Exact zeros in W with Sign(0) = q0: q0 = 0 or 0.5 cannot ride on the 1-bit operand and takes the fp32 signs."""
    xs, ws, pad, stride, dil, group = (2, 4, 9, 9), (6, 2, 3, 3), (1, 1), (1, 1), (1, 1), 2
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 43)
    W.ravel()[::4] = 0.0
    _, Wb, alpha = oracle.binary_weight_convolution(x, W, None, pad, stride, dil, group, q0)
    rdx, rdw, rdb = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, q0)
    gdx, gdw, gdb = kernels.binary_convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), _dev(Wb, dev),
                                                        _dev(alpha, dev), pad, stride, dil, group, q0)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT * 4


def test_convolution_backward_accumulates_and_skips(dev):
    xs, ws, pad, stride, dil, group = (3, 6, 8, 9), (8, 3, 3, 2), (1, 1), (2, 1), (1, 1), 2
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 44)
    alpha = np.abs(W).reshape(ws[0], -1).mean(1).astype(np.float32)
    rng = np.random.RandomState(5)
    odx, odw, odb = rng.randn(*xs).astype(np.float32), rng.randn(*ws).astype(np.float32), rng.randn(ws[0]).astype(
        np.float32)
    rdx, rdw, rdb = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0, dx=odx, dW=odw,
                                                       db=odb)
    d = lambda a: _dev(a, dev)
    gdx, gdw, gdb = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0,
                                                        dx=d(odx), dW=d(odw), db=d(odb))
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT
    only = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0,
                                               want=(True, False, False))
    assert only[1] is None and only[2] is None
    first = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0)[0]
    assert max_rel_err(to_np(only[0]), first) <= TIGHT


def test_input_gradient_as_a_convolution_accumulates(dev):
    """The same with 32 output channels per group and unit stride (the input gradient as a binary convolution of dy):
    accumulation into dx, and dx alone."""
    xs, ws, pad, stride, dil, group = (3, 6, 8, 9), (64, 3, 3, 2), (1, 1), (1, 1), (1, 1), 2
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 45)
    alpha = np.abs(W).reshape(ws[0], -1).mean(1).astype(np.float32)
    odx = np.random.RandomState(6).randn(*xs).astype(np.float32)
    rdx, _, _ = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0, dx=odx)
    d = lambda a: _dev(a, dev)
    gdx, gdw, gdb = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0,
                                                        dx=d(odx), want=(True, False, False))
    assert gdw is None and gdb is None
    assert max_rel_err(to_np(gdx), rdx) <= TIGHT
    first = oracle.binary_convolution_backward(dy, x, W, None, pad, stride, dil, group, 1.0)[0]
    only = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, None, pad, stride, dil, group, 1.0,
                                               want=(True, False, False))
    assert max_rel_err(to_np(only[0]), first) <= TIGHT


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", [
    ((8, 3, 64, 64), (48, 3, 5, 5), (2, 2), (1, 1), (1, 1), 1),        # 75 columns: two tiles, the second partly empty
    ((16, 3, 32, 32), (32, 3, 3, 3), (1, 1), (1, 1), (1, 1), 1),       # very few weights: sums per (channel pair, tap)
    ((40, 1, 28, 28), (16, 1, 5, 5), (0, 0), (1, 1), (1, 1), 1),       # ... of 25 taps, one input channel
    ((4, 3, 150, 150), (24, 3, 7, 7), (3, 3), (2, 2), (1, 1), 1),      # the first layer of an image network
    ((4, 64, 72, 72), (72, 32, 3, 3), (1, 1), (1, 1), (1, 1), 2),      # two groups, 36 channels each
    ((3, 8, 90, 80), (70, 8, 3, 2), (1, 0), (1, 1), (2, 1), 1),        # 70 channels: two tiles of channels
])
def test_weight_gradient_of_few_weights_under_many_windows(dev, xs, ws, pad, stride, dil, group):
    """16384 windows or more and at most 65536 weights per group: dW comes from fp32 kernels that read dy and x
    directly (tiles of 64 x 64 weights, or sums per thread where the weights are very few; partial results per run of
    windows, added in order); the input gradient of at most four input channels is a gather; against the oracle, with accumulation, alone and
    together with dx and db, for the real-weight and the binary layers."""
    x, W, dy = _data(xs, ws, pad, stride, dil, group, 46)
    d = lambda a: _dev(a, dev)
    rdx, rdw, rdb = oracle.convolution_backward(dy, x, W, pad, stride, dil, group)
    gdx, gdw, gdb = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT
    only = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group, want=(False, True, False))
    assert only[0] is None and only[2] is None and max_rel_err(to_np(only[1]), rdw) <= TIGHT
    again = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group, want=(False, True, False))
    assert np.array_equal(to_np(again[1]), to_np(only[1]))          # the same from run to run
    old = np.random.RandomState(7).randn(*ws).astype(np.float32)
    acc = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group, dW=d(old), want=(False, True, False))
    assert max_rel_err(to_np(acc[1]), rdw + old) <= TIGHT
    alpha = np.abs(W).reshape(ws[0], -1).mean(1).astype(np.float32)
    ref = oracle.binary_convolution_backward(dy, x, W, alpha, pad, stride, dil, group, 1.0)
    got = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(alpha), pad, stride, dil, group, 1.0)
    for g_, r_ in zip(got, ref):
        assert max_rel_err(to_np(g_), r_) <= TIGHT


def test_config4_backward(dev):
    """Benchmark configuration 4 shape (x [32,256,14,14], W [256,256,3,3], stride 1, pad 1): the oracle covers 2 of the 32
    samples for dx (samples are independent); dW and db of all 32 are checked against torch's float64 autograd on
    the CPU."""
    import torch.nn.functional as tf
    rng = np.random.default_rng(313)
    x = rng.standard_normal((32, 256, 14, 14)).astype(np.float32)
    W = (rng.standard_normal((256, 256, 3, 3)) * np.sqrt(2.0 / 2304)).astype(np.float32)
    dy = rng.standard_normal((32, 256, 14, 14)).astype(np.float32)
    alpha = np.abs(W).reshape(256, -1).mean(1).astype(np.float32)
    gdx, gdw, gdb = kernels.binary_convolution_backward(_dev(dy, dev), _dev(x, dev), _dev(W, dev), None,
                                                        _dev(alpha, dev), (1, 1), (1, 1), (1, 1), 1, 1.0)
    rdx, _, _ = oracle.binary_convolution_backward(dy[:2], x[:2], W, alpha, (1, 1), (1, 1), (1, 1), 1, 1.0,
                                                   want=(True, False, False))
    assert max_rel_err(to_np(gdx)[:2], rdx) <= TIGHT
    Ws = torch.tensor(np.where(W >= 0, 1.0, -1.0) * alpha.reshape(-1, 1, 1, 1).astype(np.float64), requires_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tf.conv2d(tx, Ws, None, stride=1, padding=1).backward(torch.tensor(dy, dtype=torch.float64))
    assert max_rel_err(to_np(gdx), tx.grad.numpy()) <= TIGHT
    assert max_rel_err(to_np(gdw), Ws.grad.numpy()) <= TIGHT
    assert max_rel_err(to_np(gdb), dy.astype(np.float64).sum((0, 2, 3))) <= TIGHT
