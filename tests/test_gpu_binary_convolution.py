"""BinaryWeightConvolution / BinaryConnectConvolution on the GPU against the CPU oracle: Sign(W) bit-exact, alpha at
rel 2e-6, outputs within max|y - y_ref| / max|y_ref| <= 1e-4 (expected ~1e-6)."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TOL, TIGHT = 1e-4, 5e-6


def _dev(x, dev):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


CASES = [
    # (x shape, w shape, pad, stride, dilation, group)
    ((2, 4, 7, 7), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 4, 7, 7), (6, 2, 3, 3), (1, 0), (2, 1), (1, 2), 2),
    ((1, 3, 9, 8), (5, 3, 2, 3), (0, 2), (1, 2), (2, 1), 1),
    ((3, 2, 10), (4, 2, 3), (1,), (2,), (1,), 1),
    ((2, 2, 4, 5, 6), (3, 2, 2, 3, 2), (1, 0, 1), (1, 2, 1), (1, 1, 2), 1),
    ((2, 6, 5, 5), (6, 1, 3, 3), (1, 1), (1, 1), (1, 1), 6),
    ((4, 8, 16, 16), (16, 8, 3, 3), (1, 1), (1, 1), (1, 1), 1),        # the reference tests' own size
    ((2, 3, 4, 8, 16, 16), (16, 8, 3, 3), (1, 1), (2, 2), (1, 1), 1),  # base_axis = 3: leading axes fold into outer
    ((3, 64, 14, 14), (96, 32, 3, 3), (1, 1), (1, 1), (1, 1), 2),
    # more than 256 output channels (two column groups of the fused unfold product, the second partly empty)
    ((2, 16, 9, 9), (300, 16, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    # images of four positions: a block of 32 windows spans eight samples
    ((40, 5, 2, 2), (7, 5, 2, 2), (1, 1), (1, 1), (1, 1), 1),
    # 125 kernel taps: above the 64 the fused product's tap mask holds, so the stand-alone unfold runs
    ((1, 2, 6, 6, 6), (4, 2, 5, 5, 5), (2, 2, 2), (1, 1, 1), (1, 1, 1), 1),
    # 7 x 7 kernel, stride 2 (49 taps: the upper half of the tap mask)
    ((2, 3, 20, 20), (8, 3, 7, 7), (3, 3), (2, 2), (1, 1), 1),
    # one output position per sample: every row of a block is a segment of its own (32 per block)
    ((70, 3, 3, 3), (5, 3, 3, 3), (0, 0), (1, 1), (1, 1), 1),
    # a wide image: the input positions under a block's 32 windows (three rows of 300) exceed what the per-position
    # maxima of the fused product hold, so its rows' maxima are gathered window by window
    ((1, 2, 5, 300), (4, 2, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    # padding larger than the kernel: windows that lie wholly outside the input
    ((2, 3, 6, 6), (4, 3, 2, 2), (3, 3), (1, 1), (1, 1), 1),
    # 24 channels per group and more: the product that keeps the input positions under a block's windows in LDS and
    # contracts over (tap, channel).  One channel tile; stride 2 with two column groups; 48 channels (padded to 64),
    # dilation 2 and rows of 40 outputs (a block's 32 windows cross rows of the map); one and three spatial
    # dimensions; groups; windows wholly outside the input; one window per sample; tiny maps
    ((2, 32, 9, 9), (40, 32, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 64, 12, 10), (300, 64, 3, 3), (1, 1), (2, 2), (1, 1), 1),
    ((2, 48, 7, 40), (16, 48, 3, 3), (1, 2), (1, 1), (2, 2), 1),
    ((3, 32, 50), (8, 32, 5), (2,), (1,), (1,), 1),
    ((1, 32, 4, 5, 6), (8, 32, 2, 3, 2), (1, 0, 1), (1, 2, 1), (1, 1, 2), 1),
    ((2, 128, 8, 8), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1), 2),
    ((2, 32, 6, 6), (4, 32, 2, 2), (3, 3), (1, 1), (1, 1), 1),
    ((70, 32, 3, 3), (5, 32, 3, 3), (0, 0), (1, 1), (1, 1), 1),
    ((40, 32, 2, 2), (7, 32, 2, 2), (1, 1), (1, 1), (1, 1), 1),
    ((1, 24, 5, 70), (4, 24, 1, 7), (0, 3), (1, 3), (1, 1), 1),
    # the positions under a block (three rows of 70) times 96 channels: more than a wavefront keeps in registers
    ((1, 96, 5, 70), (8, 96, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    # nine channel tiles (alpha summed from more than eight partial sums)
    ((1, 288, 6, 6), (8, 288, 3, 3), (1, 1), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
@pytest.mark.parametrize("bias", [False, True])
def test_binary_weight_convolution_matches_oracle(dev, xs, ws, pad, stride, dil, group, bias):
    rng = np.random.RandomState(313)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32) if bias else None
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, pad, stride, dil, group, 1.0)
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), None if b is None else _dev(b, dev),
                                                     pad, stride, dil, group)
    assert tuple(y.shape) == ref_y.shape
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CASES)
def test_binary_connect_convolution_matches_oracle(dev, xs, ws, pad, stride, dil, group):
    rng = np.random.RandomState(7)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)
    ref_y, ref_Wb = oracle.binary_connect_convolution(x, W, b, pad, stride, dil, group, 1.0)
    y, Wb = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), pad, stride, dil, group)
    assert bits_equal(to_np(Wb), ref_Wb)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT


@pytest.mark.parametrize("channels", [4, 64])
@pytest.mark.parametrize("q0", [0.0, -1.0, 0.5])
def test_convolution_quantize_zero_to_with_zero_weights(dev, q0, channels):
    rng = np.random.RandomState(3)
    x = rng.randn(2, channels, 9, 9).astype(np.float32)
    W = (rng.randn(6, channels // 2, 3, 3) * 0.05).astype(np.float32)
    W.ravel()[::4] = 0.0
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, None, (1, 1), (1, 1), (1, 1), 2, q0)
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), None, (1, 1), (1, 1), (1, 1), 2, q0)
    assert bits_equal(to_np(Wb), ref_Wb)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT * 4
    ref_y, _ = oracle.binary_connect_convolution(x, W, None, (1, 1), (1, 1), (1, 1), 2, q0)
    y, _ = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), None, (1, 1), (1, 1), (1, 1), 2, q0)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT * 4


def _same_non_finite(y, ref):
    """NaN, +Inf and -Inf at the same places, the finite outputs within the products' tolerance."""
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert np.array_equal(np.isposinf(y), np.isposinf(ref))
    assert np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin.any() and (~fin).any()
    assert np.abs(y[fin] - ref[fin]).max() / np.abs(ref[fin]).max() <= TIGHT


# (x shape, W shape, pad, stride, dilation, group): the product that keeps input positions in LDS (32 channels), the
# gathering product (8 channels), the unfolded digit matrix (a kernel of 81 taps), and groups / stride / padding
NON_FINITE_CASES = [
    ((2, 32, 9, 9), (6, 32, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 64, 9, 9), (300, 32, 3, 3), (1, 1), (1, 1), (1, 1), 2),
    ((2, 8, 9, 9), (6, 8, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 8, 9, 9), (6, 4, 3, 3), (0, 2), (2, 1), (1, 2), 2),
    ((2, 4, 12, 12), (5, 4, 9, 9), (4, 4), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", NON_FINITE_CASES)
@pytest.mark.parametrize("with_bias", [False, True])
def test_window_with_a_non_finite_value(dev, xs, ws, pad, stride, dil, group, with_bias):
    """An Inf or NaN in x: the reference's product propagates it output by output (convolution.cpp:185-193:
    Inf * w = +-Inf by the weight's sign, Inf - Inf = NaN, NaN anywhere = NaN), and so do the windows recomputed here;
    two infinities under the same windows make some outputs NaN and others +-Inf.  All other outputs are the ones of
    the clean input, bit for bit."""
    rng = np.random.RandomState(5)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32) if with_bias else None
    bd = _dev(b, dev) if with_bias else None
    clean, _, _ = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), bd, pad, stride, dil, group)
    x[1, 3, 4, 5] = np.inf
    x[1, 2, 4, 6] = np.inf
    x[1, 1, 7, 2] = -np.inf
    x[0, 0, 0, 0] = np.nan
    with np.errstate(invalid="ignore", over="ignore"):
        ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, pad, stride, dil, group, 1.0)
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), bd, pad, stride, dil, group)
    y, clean = to_np(y), to_np(clean)
    _same_non_finite(y, ref_y)
    touched = ~np.isfinite(ref_y).all(axis=1, keepdims=True) | ~np.isfinite(y).all(axis=1, keepdims=True)
    keep = np.broadcast_to(~touched, y.shape)
    assert bits_equal(y[keep], clean[keep])
    with np.errstate(invalid="ignore", over="ignore"):
        ref_y, _ = oracle.binary_connect_convolution(x, W, b, pad, stride, dil, group, 1.0)
    y, _ = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), bd, pad, stride, dil, group)
    _same_non_finite(to_np(y), ref_y)


def test_wide_range_inside_the_positions_under_a_block(dev):
    """The product over input positions held in LDS rounds x to a multiple of 2^-28 of the largest magnitude among the
    positions under a block's (at most 32) windows: |y - y64| <= K * 2^-29 * max|x| (+ the fp32 rounding of y), shown
    on BinaryConnectConvolution (no alpha).  One position 2^12 and one 2^20 times the rest: the bound holds, and
    windows that do not touch them still agree with float64 to 1e-4 of their own largest output in the first case."""
    rng = np.random.RandomState(11)
    W = (rng.randn(16, 32, 3, 3) * 0.05).astype(np.float32)
    s64 = torch.from_numpy(np.where(W < 0, -1.0, 1.0))
    for factor in (2.0 ** 12, 2.0 ** 20):
        x = rng.randn(1, 32, 14, 14).astype(np.float32)
        x[0, :, 3, 3] *= np.float32(factor)
        y, _ = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), None, (1, 1), (1, 1), (1, 1), 1)
        y = to_np(y).astype(np.float64)
        y64 = torch.nn.functional.conv2d(torch.from_numpy(x).double(), s64, None, 1, 1).numpy()
        bound = 288 * 2.0 ** -29 * np.abs(x).max() + 2.0 ** -24 * np.abs(y64)
        assert (np.abs(y - y64) <= bound).all()
        far = np.ones((14, 14), bool)
        far[2:5, 2:5] = False
        err = np.abs(y - y64)[0][:, far].max() / np.abs(y64)[0][:, far].max()
        print("outlier x%g: error of the windows away from it / their largest output = %.2e" % (factor, err))
        if factor == 2.0 ** 12:
            assert err <= 1e-4


def test_config4_resnet_stage(dev):
    """Benchmark configuration 4: x [32,256,14,14] ~ N(0,1), W [256,256,3,3] ~ N(0, 2/2304), stride 1, pad 1, zero bias.
    The oracle is run on 4 of the 32 samples (convolution is independent per sample); all 32 are checked against
    torch's float64 convolution on the same binarized weights."""
    rng = np.random.default_rng(313)
    x = rng.standard_normal((32, 256, 14, 14), dtype=np.float32)
    W = rng.standard_normal((256, 256, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / 2304))
    b = np.zeros(256, np.float32)
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), (1, 1), (1, 1), (1, 1))
    yc, Wbc = kernels.binary_connect_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), (1, 1), (1, 1), (1, 1))
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x[:4], W, b, (1, 1), (1, 1), (1, 1), 1, 1.0)
    ref_yc, _ = oracle.binary_connect_convolution(x[:4], W, b, (1, 1), (1, 1), (1, 1), 1, 1.0)
    assert bits_equal(to_np(Wb), ref_Wb) and bits_equal(to_np(Wbc), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    assert max_rel_err(to_np(y)[:4], ref_y) <= TOL and max_rel_err(to_np(yc)[:4], ref_yc) <= TOL
    s64 = torch.from_numpy(ref_Wb).double()
    full = torch.nn.functional.conv2d(torch.from_numpy(x).double(), s64, None, 1, 1).numpy()
    a64 = np.abs(W.astype(np.float64)).reshape(256, -1).mean(1).reshape(1, -1, 1, 1)
    assert max_rel_err(to_np(yc), full) <= TIGHT
    assert max_rel_err(to_np(y), full * a64) <= TIGHT


@pytest.mark.parametrize("xs,ws,stride", [
    ((4, 64, 56, 56), (64, 64, 3, 3), 1),      # rows of 56 outputs: a block's 32 windows cross rows; 64 of 256 channels
    ((4, 128, 28, 28), (128, 128, 3, 3), 1),
    ((4, 512, 7, 7), (512, 512, 3, 3), 1),     # two column groups, 16 channel tiles, tiles of four rows of the map
    ((4, 64, 56, 56), (128, 64, 3, 3), 2),     # a strided stage transition
    ((3, 256, 14, 14), (512, 256, 1, 1), 1),   # 1 x 1 kernel: one tap
])
def test_residual_network_stages_against_float64(dev, xs, ws, stride):
    """The other stages of the network benchmark configuration 4 is taken from, a few samples each, against torch's
    float64 convolution on the binarized weights."""
    rng = np.random.default_rng(99)
    x = rng.standard_normal(xs, dtype=np.float32)
    W = rng.standard_normal(ws, dtype=np.float32) * np.float32(np.sqrt(2.0 / np.prod(ws[1:])))
    b = rng.standard_normal(ws[0], dtype=np.float32)
    pad = ws[2] // 2
    y, Wb, alpha = kernels.binary_weight_convolution(_dev(x, dev), _dev(W, dev), _dev(b, dev), (pad, pad),
                                                     (stride, stride), (1, 1))
    s64 = torch.from_numpy(np.where(W < 0, -1.0, 1.0))
    a64 = np.abs(W.astype(np.float64)).reshape(ws[0], -1).mean(1).reshape(1, -1, 1, 1)
    full = torch.nn.functional.conv2d(torch.from_numpy(x).double(), s64, None, stride, pad).numpy()
    ref = full * a64 + b.astype(np.float64).reshape(1, -1, 1, 1)
    assert bits_equal(to_np(Wb), np.where(W < 0, -1.0, 1.0).astype(np.float32))
    np.testing.assert_allclose(to_np(alpha).ravel(), a64.ravel(), rtol=2e-6)
    assert max_rel_err(to_np(y), ref) <= TIGHT


def test_convolution_argument_errors(dev):
    x = _dev(np.zeros((1, 4, 5, 5), np.float32), dev)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.binary_weight_convolution(x, _dev(np.zeros((6, 4, 7, 7), np.float32), dev))
    assert ei.value.code == kernels.ERR_VALUE
    with pytest.raises(kernels.KernelError) as ei:
        kernels.binary_connect_convolution(x, _dev(np.zeros((6, 2, 3, 3), np.float32), dev), group=3)
    assert ei.value.code == kernels.ERR_VALUE


@pytest.mark.parametrize("channels,q0,zeros", [(32, 1.0, False), (32, 0.0, True), (8, 1.0, False), (8, 0.0, True)])
def test_forward_and_backward_replay_in_a_hip_graph(dev, channels, q0, zeros):
    """The convolution's forward and backward captured once and replayed on new inputs, for the product on input
    positions held in LDS (32 channels) and the gathering product (8), with quantize_zero_to decided on the device:
    every replay gives the eager call's bits (eager work and synchronisations run between the replays)."""
    rng = np.random.RandomState(5)
    xs, ws = (2, channels, 9, 9), (40, channels, 3, 3)
    Wh = (rng.randn(*ws) * 0.05).astype(np.float32)
    if zeros:
        Wh.ravel()[::7] = 0.0
    W = _dev(Wh, dev)
    x = torch.empty(xs, device=dev)
    dy = torch.empty((2, 40, 9, 9), device=dev)

    def step():
        y, Wb, alpha = kernels.binary_weight_convolution(x, W, None, (1, 1), (1, 1), (1, 1), 1, q0)
        dx, dW, db = kernels.binary_convolution_backward(dy, x, W, Wb, alpha, (1, 1), (1, 1), (1, 1), 1, q0)
        return y, dx, dW, db

    x.copy_(_dev(rng.randn(*xs).astype(np.float32), dev))
    dy.copy_(_dev(rng.randn(2, 40, 9, 9).astype(np.float32), dev))
    step()                                   # first call outside the capture (one-time kernel attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for i in range(3):
        x.copy_(_dev((rng.randn(*xs) * (i + 1)).astype(np.float32), dev))
        dy.copy_(_dev(rng.randn(2, 40, 9, 9).astype(np.float32), dev))
        graph.replay()
        torch.cuda.synchronize()
        got = [to_np(o).copy() for o in outs]
        eager = step()
        torch.cuda.synchronize()
        for g, e, name in zip(got, eager, ("y", "dx", "dW", "db")):
            assert bits_equal(g, to_np(e)), "replay %d: %s differs from the eager result" % (i, name)
        ref_y, _, _ = oracle.binary_weight_convolution(to_np(x), Wh, None, (1, 1), (1, 1), (1, 1), 1, q0)
        assert max_rel_err(got[0], ref_y) <= TOL
