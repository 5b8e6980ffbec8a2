"""GPU parity of the quantizer backward passes against the CPU oracle: bit-exact for dx (the masks and the STE are
elementwise), float64 tolerance for the MinMaxQuantize range gradients (sums)."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, first_mismatch, to_np

pytestmark = pytest.mark.gpu


def _dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _rand(shape, seed, scale=1.0):
    return (np.random.RandomState(seed).randn(*shape) * scale).astype(np.float32)


@pytest.mark.parametrize("shape", [(3,), (5, 37), (256, 1031), (4, 8, 16, 16)])
@pytest.mark.parametrize("sign,n,delta", [(True, 8, 2.0 ** -4), (False, 4, 0.1)])
@pytest.mark.parametrize("fine", [True, False])
def test_fixed_point_backward(dev, shape, sign, n, delta, fine):
    x, dy, old = _rand(shape, 1, 5.0), _rand(shape, 2), _rand(shape, 3)
    nn = n - 1 if sign else n
    x.ravel()[:2] = [(2 ** nn - 1) * delta, 0.0]
    ref = oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, fine)
    got = to_np(kernels.fixed_point_quantize_backward(_dev(dy, dev), _dev(x, dev), sign, n, delta, fine))
    assert bits_equal(got, ref), first_mismatch(got, ref)
    ref = oracle.fixed_point_quantize_backward(dy, x, sign, n, delta, fine, dx=old)
    got = to_np(kernels.fixed_point_quantize_backward(_dev(dy, dev), _dev(x, dev), sign, n, delta, fine,
                                                      dx=_dev(old, dev)))
    assert bits_equal(got, ref), first_mismatch(got, ref)


@pytest.mark.parametrize("shape", [(7,), (64, 513), (512, 512, 3, 3)])
@pytest.mark.parametrize("sign,with_zero,n,m", [(True, True, 4, 1), (False, True, 4, 0), (True, False, 3, -2),
                                                (False, False, 2, 3)])
def test_pow2_backward(dev, shape, sign, with_zero, n, m):
    x, dy, old = _rand(shape, 5, 2.0 ** m), _rand(shape, 6), _rand(shape, 7)
    # the sqrt(2) window of the top level, specials
    top = np.float32(2.0 ** m * np.sqrt(2.0))
    probes = [top, np.nextafter(top, np.float32(0)), np.nextafter(top, np.float32(np.inf)), 0.0, -0.0, np.inf, -np.inf,
              np.nan]
    x.ravel()[:min(len(probes), x.size)] = probes[:x.size]
    for fine in (True, False):
        ref = oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, fine)
        got = to_np(kernels.pow2_quantize_backward(_dev(dy, dev), _dev(x, dev), sign, with_zero, n, m, fine))
        assert bits_equal(got, ref), first_mismatch(got, ref)
        ref = oracle.pow2_quantize_backward(dy, x, sign, with_zero, n, m, fine, dx=old)
        got = to_np(kernels.pow2_quantize_backward(_dev(dy, dev), _dev(x, dev), sign, with_zero, n, m, fine,
                                                   dx=_dev(old, dev)))
        assert bits_equal(got, ref), first_mismatch(got, ref)


def test_pow2_backward_all_binade_cuts(dev):
    """Every value adjacent to the libm-defined cut of the top level, for several m."""
    for m in (-20, -3, 0, 1, 10):
        centre = np.float32(2.0 ** m * np.sqrt(2.0))
        xs = [centre]
        for _ in range(40):
            xs.append(np.nextafter(xs[-1], np.float32(np.inf)))
        lo = centre
        for _ in range(40):
            lo = np.nextafter(lo, np.float32(0))
            xs.append(lo)
        x = np.array(xs + [-v for v in xs], np.float32)
        dy = np.ones_like(x)
        ref = oracle.pow2_quantize_backward(dy, x, True, True, 8, m, True)
        got = to_np(kernels.pow2_quantize_backward(_dev(dy, dev), _dev(x, dev), True, True, 8, m, True))
        assert bits_equal(got, ref), (m, first_mismatch(got, ref))


@pytest.mark.parametrize("xshape,qshape", [((4, 6, 5, 3), (1, 1, 1, 1)), ((4, 6, 5, 3), (1, 6, 1, 1)),
                                           ((4, 6, 5, 3), (4, 1, 1, 1)), ((16, 8, 32, 32), (1, 8, 1, 1)),
                                           ((2, 3, 7), (1, 1, 1)), ((64, 1000), (1, 1000)),
                                           ((5, 7, 9), (5, 1, 9)), ((3, 4, 5, 6), (1, 4, 1, 6)),
                                           ((6, 300, 7), (6, 1, 7)), ((2, 3, 1, 4, 5), (2, 1, 1, 4, 1)),
                                           # one pass over dy and x: rows of a channel, one range, lanes along the
                                           # kept innermost axis (single columns and quads), ranges per column
                                           ((8, 16, 24, 24), (8, 16, 1, 1)), ((3, 5, 40, 64), (1, 5, 1, 1)),
                                           ((33, 1025), (1, 1)), ((40, 70, 130), (1, 1, 1)),
                                           ((6, 10, 8, 12), (1, 10, 1, 12)), ((4, 10, 100), (4, 1, 100)),
                                           ((300, 520), (1, 520)), ((40, 33, 20), (1, 1, 20)),
                                           ((7, 3, 5, 9), (1, 1, 5, 9)), ((5000, 3), (1, 3)),
                                           # the innermost axis reduced in short runs
                                           ((6, 40, 30, 56), (1, 40, 30, 1)), ((9, 3, 50, 12), (9, 1, 50, 1)),
                                           ((5, 3, 7, 300), (5, 1, 7, 1)), ((4, 6, 10, 70), (1, 6, 10, 1)),
                                           ((700, 9, 5), (1, 9, 1)), ((2, 3, 2000, 6), (2, 1, 2000, 1)),
                                           ((8, 16, 27, 27), (1, 16, 1, 1)), ((3, 4, 4097), (3, 4, 1))])
@pytest.mark.parametrize("fine", [True, False])
def test_min_max_backward(dev, xshape, qshape, fine):
    x, dy = _rand(xshape, 11, 3.0), _rand(xshape, 12)
    qr_min = np.full(qshape, -2.0, np.float32) + _rand(qshape, 13, 0.1)
    qr_max = np.full(qshape, 2.5, np.float32) + _rand(qshape, 14, 0.1)
    ql_min, ql_max = np.zeros(qshape, np.float32), np.full(qshape, 255.0, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, 0.999, False, False, 0.01)
    rdx, rmin, rmax = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, fine, False, False)
    d = lambda a: _dev(a, dev)
    gdx, gmin, gmax = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(ql_min), d(ql_max), d(scale), fine,
                                                        False, False)
    assert bits_equal(to_np(gdx), rdx), first_mismatch(to_np(gdx), rdx)
    axes = tuple(i for i in range(len(xshape)) if qshape[i] == 1)
    denom = np.abs(dy).astype(np.float64).sum(axis=axes, keepdims=True) + 1e-30
    assert (np.abs(to_np(gmin) - rmin.astype(np.float64)) / denom).max() <= 2e-6
    assert (np.abs(to_np(gmax) - rmax.astype(np.float64)) / denom).max() <= 2e-6
    # accumulation, and partial propagation
    odx, omin, omax = _rand(xshape, 15), _rand(qshape, 16), _rand(qshape, 17)
    rdx2, rmin2, rmax2 = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, fine, False, False,
                                                          dx=odx, g_qr_min=omin, g_qr_max=omax)
    gdx2, gmin2, gmax2 = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(ql_min), d(ql_max), d(scale),
                                                           fine, False, False, dx=d(odx), g_qr_min=d(omin),
                                                           g_qr_max=d(omax))
    assert bits_equal(to_np(gdx2), rdx2)
    # (the sums are formed in a fixed order that is not the reference's: their error is relative to the sum of |dy|)
    assert (np.abs(to_np(gmin2) - rmin2.astype(np.float64)) / (denom + np.abs(omin))).max() <= 2e-6
    assert (np.abs(to_np(gmax2) - rmax2.astype(np.float64)) / (denom + np.abs(omax))).max() <= 2e-6
    only_max = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(ql_min), d(ql_max), d(scale), fine,
                                                 False, False, want_x=False, want_min=False)
    assert only_max[0] is None and only_max[1] is None
    assert (np.abs(to_np(only_max[2]) - rmax.astype(np.float64)) / denom).max() <= 2e-6


def _random_axis_patterns(count, seed):
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        nd = int(rng.randint(1, 6))
        xshape = tuple(int(v) for v in rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 130], size=nd))
        if int(np.prod(xshape)) > 300000:
            continue
        keep = rng.rand(nd) < 0.4
        out.append((xshape, tuple(s if k else 1 for s, k in zip(xshape, keep))))
    return out


@pytest.mark.parametrize("xshape,qshape", _random_axis_patterns(40, 578))
def test_min_max_backward_random_axis_patterns(dev, xshape, qshape):
    """Ranks 1 to 5 with every axis kept or reduced at random: the input gradient bit for bit, the range gradients
    (sums in a fixed order of their own) relative to the sum of |dy| over the reduced axes."""
    print("shapes", xshape, qshape, flush=True)
    x, dy = _rand(xshape, 21, 3.0), _rand(xshape, 22)
    qr_min = np.full(qshape, -2.0, np.float32) + _rand(qshape, 23, 0.1)
    qr_max = np.full(qshape, 2.5, np.float32) + _rand(qshape, 24, 0.1)
    ql_min, ql_max = np.zeros(qshape, np.float32), np.full(qshape, 255.0, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, 0.999, False, False, 0.01)
    d = lambda a: _dev(a, dev)
    axes = tuple(i for i in range(len(xshape)) if qshape[i] == 1)
    denom = np.abs(dy).astype(np.float64).sum(axis=axes, keepdims=True) + 1e-30
    for fine in (True, False):
        rdx, rmin, rmax = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, fine, False, False)
        gdx, gmin, gmax = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(ql_min), d(ql_max), d(scale),
                                                            fine, False, False)
        assert bits_equal(to_np(gdx), rdx), first_mismatch(to_np(gdx), rdx)
        assert (np.abs(to_np(gmin) - rmin.astype(np.float64)) / denom).max() <= 2e-6
        assert (np.abs(to_np(gmax) - rmax.astype(np.float64)) / denom).max() <= 2e-6


@pytest.mark.parametrize("xshape,qshape", [((3, 5, 40, 64), (1, 5, 1, 1)), ((6, 10, 8, 12), (1, 10, 1, 12)),
                                           ((300, 520), (1, 520)), ((5, 7, 9), (5, 1, 9)), ((4, 6, 5, 3), (1, 6, 1, 1)),
                                           ((9, 3, 50, 12), (9, 1, 50, 1)), ((4, 6, 10, 70), (1, 6, 10, 1))])
@pytest.mark.parametrize("accumulate", [False, True])
def test_min_max_backward_input_gradient_alone(dev, xshape, qshape, accumulate):
    """Ranges that follow the statistics of x (x_min_max) are not learnt: only dx is formed, by the same one-pass
    kernels without their sums, and the range gradients passed in stay as they are."""
    x, dy = _rand(xshape, 31, 3.0), _rand(xshape, 32)
    qr_min = np.full(qshape, -2.0, np.float32) + _rand(qshape, 33, 0.1)
    qr_max = np.full(qshape, 2.5, np.float32) + _rand(qshape, 34, 0.1)
    ql_min, ql_max = np.zeros(qshape, np.float32), np.full(qshape, 255.0, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, 0.999, True, False, 0.01)
    odx = _rand(xshape, 35) if accumulate else None
    rdx, _, _ = oracle.min_max_quantize_backward(dy, x, qmn, qmx, ql_min, ql_max, scale, True, True, False, dx=odx)
    d = lambda a: _dev(a, dev)
    keep_min, keep_max = d(np.full(qshape, 7.0, np.float32)), d(np.full(qshape, 9.0, np.float32))
    gdx, gmin, gmax = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(ql_min), d(ql_max), d(scale), True,
                                                        True, False, dx=d(odx) if accumulate else None,
                                                        g_qr_min=keep_min, g_qr_max=keep_max)
    assert bits_equal(to_np(gdx), rdx), first_mismatch(to_np(gdx), rdx)
    assert (to_np(gmin) == 7.0).all() and (to_np(gmax) == 9.0).all()


@pytest.mark.parametrize("x_min_max,ema", [(True, False), (False, True)])
def test_min_max_backward_statistics_modes_leave_range_gradients(dev, x_min_max, ema):
    x, dy = _rand((2, 3, 4, 4), 21), _rand((2, 3, 4, 4), 22)
    q = lambda v: np.full((1, 1, 1, 1), v, np.float32)
    _, qmn, qmx, scale = oracle.min_max_quantize(x, q(-1), q(1), q(0), q(255), 0.999, x_min_max, ema, 0.01)
    d = lambda a: _dev(a, dev)
    sent_min, sent_max = d(q(7.0)), d(q(9.0))
    gdx, gmin, gmax = kernels.min_max_quantize_backward(d(dy), d(x), d(qmn), d(qmx), d(q(0)), d(q(255)), d(scale), True,
                                                        x_min_max, ema, g_qr_min=sent_min, g_qr_max=sent_max)
    rdx, _, _ = oracle.min_max_quantize_backward(dy, x, qmn, qmx, q(0), q(255), scale, True, x_min_max, ema)
    assert bits_equal(to_np(gdx), rdx)
    assert to_np(gmin).item() == 7.0 and to_np(gmax).item() == 9.0


@pytest.mark.parametrize("sign,n,delta", [(True, 8, 2.0 ** -4), (False, 5, 0.3)])
def test_fixed_point_backward_every_fp32_value(dev, sign, n, delta):
    """The fine-grained STE mask of fixed_point_quantize.cpp:84-99 for all 2^32 bit patterns of x (dy = 3): dx = dy
    inside [min, max] (and for NaN, which fails both comparisons), 0 outside."""
    nn = n - 1 if sign else n
    mx = float(np.float32((2.0 ** nn - 1) * float(np.float32(delta))))
    mn = -mx if sign else 0.0
    chunk = 1 << 27
    dy = torch.full((chunk,), 3.0, device=dev)
    for start in range(0, 1 << 32, chunk):
        lo = start - (1 << 32) if start >= (1 << 31) else start
        x = torch.arange(lo, lo + chunk, dtype=torch.int32, device=dev).view(torch.float32)
        dx = kernels.fixed_point_quantize_backward(dy, x, sign, n, delta, True)
        ref = torch.where((x > mx) | (x < mn), torch.zeros_like(dy), dy)
        assert bool((dx == ref).all()), "chunk starting at bits %#x" % start


@pytest.mark.parametrize("sign,with_zero,n,m", [(True, True, 4, 1), (False, False, 6, 3)])
def test_pow2_backward_every_normal_fp32_value(dev, sign, with_zero, n, m):
    """The fine-grained STE mask of pow2_quantize.cpp:97-125 for every normal x farther than 64 ulp from a cut
    2^(k + 1/2) (the neighbourhoods of the cuts are compared with the host libm in the test above): 0 where
    2^round(log2|x|) exceeds 2^m, and for negative x of the unsigned form."""
    p_max = float(2.0 ** m)
    chunk = 1 << 27
    dy = torch.full((chunk,), -2.5, device=dev)
    for start in range(0, 1 << 32, chunk):
        lo = start - (1 << 32) if start >= (1 << 31) else start
        bits = torch.arange(lo, lo + chunk, dtype=torch.int32, device=dev)
        x = bits.view(torch.float32)
        dx = kernels.pow2_quantize_backward(dy, x, sign, with_zero, n, m, True)
        q = torch.exp2(torch.round(torch.log2(x.abs().double())))
        c = q <= p_max
        if not sign:
            c = c & ~(x < 0)
        ref = torch.where(c, dy, torch.zeros_like(dy))
        mant, expo = bits & 0x7fffff, (bits >> 23) & 0xff
        checked = (expo > 0) & (expo < 255) & ((mant - 0x3504f3).abs() > 64)
        assert bool(((dx == ref) | ~checked).all()), "chunk starting at bits %#x" % start
