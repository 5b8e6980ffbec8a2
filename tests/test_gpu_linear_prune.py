"""QuantizeLinear / DequantizeLinear / Prune on the GPU against the CPU oracle: bit-exact (every step of the
reference chain is a separately rounded fp32 operation; Prune's threshold is an order statistic)."""
import ctypes

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


SHAPES = [
    # (x shape, scale shape, zero-point shape)
    ((3, 5, 7), (1, 1, 1), (1, 1, 1)),
    ((3, 5, 7), (1, 5, 1), (1, 5, 1)),
    ((3, 5, 8), (3, 1, 1), (1, 1, 8)),
    ((3, 5, 8), (3, 5, 8), (1, 5, 1)),
    ((4, 16, 6, 6), (1, 16, 1, 1), (1, 16, 1, 1)),
    ((2, 3, 4, 5, 6, 8), (2, 1, 4, 1, 6, 1), (1, 3, 1, 5, 1, 8)),
    ((64, 4096), (1, 1), (1, 1)),
    ((64, 4096), (1, 4096), (1, 1)),
    ((1000,), (1,), (1,)),
    ((1, 1), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("xs,ss,zs", SHAPES)
@pytest.mark.parametrize("mode,narrow,dtype", [("HALF_AWAY_FROM_ZERO", False, 1), ("HALF_TO_EVEN", True, 1),
                                               ("HALF_TO_EVEN", False, 2), ("HALF_AWAY_FROM_ZERO", True, 2)])
def test_quantize_linear(dev, xs, ss, zs, mode, narrow, dtype):
    x = _rand(xs, 1, 60.0)
    x.ravel()[:6] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5][:min(6, x.size)]
    scale = (np.abs(_rand(ss, 2)) + 0.25).astype(np.float32)
    if int(np.prod(ss)) == 1:
        scale[...] = 0.5
    zp = _rand(zs, 3, 40.0)
    ref, ref_zp = oracle.quantize_linear(x, scale, zp, mode, narrow, dtype)
    dzp = _dev(zp, dev)
    y = kernels.quantize_linear(_dev(x, dev), _dev(scale, dev), dzp, mode, narrow, dtype)
    assert bits_equal(to_np(y), ref)
    assert bits_equal(to_np(dzp), ref_zp)                          # rounded and saturated in place


@pytest.mark.parametrize("mode", ["HALF_AWAY_FROM_ZERO", "HALF_TO_EVEN"])
@pytest.mark.parametrize("scale,zp", [(0.3, 2.5), (0.0371, -3.5), (7.0, 300.0), (1e-30, 0.49), (3e38, -0.5)])
@pytest.mark.parametrize("n", [1, 5, 4096, 1 << 18, (1 << 18) + 3])
def test_quantize_linear_one_scale_one_zero_point(dev, mode, scale, zp, n):
    """Per-tensor parameters (one scale, one unrounded zero point, handled inside the main launch): ties of the zero
    point, saturating zero points, scales at the ends of the range, vector and element-wise sizes."""
    with np.errstate(over='ignore'):                       # the largest scale takes some inputs to infinity
        x = _rand((n,), n % 97, 40.0 * scale if scale < 1e30 else 1e38)
        x[:min(n, 4)] = np.array([0.5, -0.5, 1.5, 2.5], np.float32)[:min(n, 4)] * np.float32(scale)
    s, z = np.full((1,), scale, np.float32), np.full((1,), zp, np.float32)
    for dtype, narrow in ((1, False), (2, True)):
        ref, ref_zp = oracle.quantize_linear(x, s, z, mode, narrow, dtype)
        dz = _dev(z, dev)
        y = kernels.quantize_linear(_dev(x, dev), _dev(s, dev), dz, mode, narrow, dtype)
        assert bits_equal(to_np(y), ref), first_mismatch(to_np(y), ref)
        assert bits_equal(to_np(dz), ref_zp)


@pytest.mark.parametrize("xs,ss,zs", SHAPES)
def test_dequantize_linear_and_backward(dev, xs, ss, zs):
    x = np.rint(_rand(xs, 4, 50.0)).astype(np.float32)
    scale = (np.abs(_rand(ss, 5)) + 0.1).astype(np.float32)
    zp = np.rint(_rand(zs, 6, 5.0)).astype(np.float32)
    y = kernels.dequantize_linear(_dev(x, dev), _dev(scale, dev), _dev(zp, dev))
    assert bits_equal(to_np(y), oracle.dequantize_linear(x, scale, zp))
    dy, old = _rand(xs, 7), _rand(xs, 8)
    for deq in (False, True):
        g = kernels.linear_quantize_backward(_dev(dy, dev), _dev(scale, dev), deq)
        assert bits_equal(to_np(g), oracle.linear_quantize_backward(dy, scale, deq))
        acc = _dev(old, dev)
        kernels.linear_quantize_backward(_dev(dy, dev), _dev(scale, dev), deq, dx=acc)
        assert bits_equal(to_np(acc), oracle.linear_quantize_backward(dy, scale, deq, dx=old))


def test_quantize_linear_rejects_bad_arguments(dev):
    x, one = _dev(np.zeros((2, 3), np.float32), dev), _dev(np.ones((1, 1), np.float32), dev)
    with pytest.raises(kernels.KernelError) as e:
        kernels.quantize_linear(x, one, one.clone(), dtype=5)
    assert e.value.code == kernels.ERR_VALUE
    with pytest.raises(kernels.KernelError) as e:
        kernels.quantize_linear(x, _dev(np.ones((2, 2), np.float32), dev), one.clone())
    assert e.value.code == kernels.ERR_VALUE


@pytest.mark.parametrize("size", [1, 7, 1000, 4097, 1 << 20])
@pytest.mark.parametrize("rate", [0.0, 0.33, 0.5, 0.9, 1.0])
def test_prune(dev, size, rate):
    x = _rand((size,), 9, 3.0)
    if size > 20:
        x[::7] = x[3]
        x[::14] = -x[3]
        x[5] = 0.0
        x[6] = -0.0
    y = kernels.prune(_dev(x, dev), rate)
    assert bits_equal(to_np(y), oracle.prune(x, rate))


@pytest.mark.parametrize("x_off,y_off", [(1, 0), (0, 3), (2, 2), (1, 3)])
def test_prune_on_views_that_are_not_16_byte_aligned(dev, x_off, y_off):
    """x or y starting at an odd multiple of four bytes (a narrowed view of a larger array): the same result, through
    32-bit accesses."""
    rng = np.random.RandomState(9)
    n = 100003
    x = rng.randn(n).astype(np.float32)
    xb = torch.zeros(n + 8, device=dev)
    xb[x_off:x_off + n] = torch.from_numpy(x).to(dev)
    yb = torch.full((n + 8,), 7.0, device=dev)
    xv, yv = xb[x_off:x_off + n], yb[y_off:y_off + n]
    assert (xv.data_ptr() % 16 != 0) or (yv.data_ptr() % 16 != 0)
    ws = torch.empty(kernels.lib().nbla_hip_prune_workspace_bytes(), dtype=torch.uint8, device=dev)
    kernels.check(kernels.lib().nbla_hip_prune_f32(kernels._p(xv), kernels._p(yv), ctypes.c_size_t(n), ctypes.c_float(0.7),
                                                   kernels._p(ws), ctypes.c_size_t(ws.numel()), None))
    assert bits_equal(to_np(yv), oracle.prune(x, 0.7))
    assert (to_np(yb[:y_off]) == 7.0).all() and (to_np(yb[y_off + n:]) == 7.0).all()


def test_prune_large_and_special_values(dev):
    """16.8 M elements (the FixedPointQuantize bench shape) with denormals and infinities; the radix select must land
    on exactly the element a full sort would."""
    rng = np.random.default_rng(313)
    x = (rng.standard_normal((256, 65536)) * 2).astype(np.float32)
    x.ravel()[:4] = [np.inf, -np.inf, 1e-42, -1e-42]
    for rate in (0.5, 0.999):
        y = kernels.prune(_dev(x, dev), rate)
        assert bits_equal(to_np(y), oracle.prune(x, rate))
    with pytest.raises(kernels.KernelError):
        kernels.prune(_dev(x[:1], dev), 1.5)


@pytest.mark.parametrize("rate", [0.3, 0.6, 0.97])
def test_prune_magnitudes_clustered_in_one_stretch(dev, rate):
    """The second selection pass keeps the keys that share the first digit with the threshold in per-block regions of
    the workspace; when those keys sit in one stretch of x (here: 1.3 M values of one binade in a row, far more than
    the blocks that read that stretch can keep) the third pass has to fall back to reading x.  Same result either
    way; the first rate puts the threshold outside the stretch, the others inside it."""
    rng = np.random.default_rng(77)
    n = 1 << 22
    x = (rng.standard_normal(n) * 0.01).astype(np.float32)
    lo = n // 3
    x[lo:lo + 1300000] = (1.0 + rng.random(1300000) * 0.12).astype(np.float32) * rng.choice([-1.0, 1.0], 1300000).astype(np.float32)
    x[lo + 1300000:] *= 1000.0
    y = kernels.prune(_dev(x, dev), rate)
    assert bits_equal(to_np(y), oracle.prune(x, rate))


def test_prune_reuses_its_workspace(dev):
    """Back-to-back calls on one workspace (histograms, tickets and chosen digits of the previous call are left in
    it), with changing sizes and rates."""
    import torch
    ws = torch.empty(kernels.lib().nbla_hip_prune_workspace_bytes(), dtype=torch.uint8, device=dev)
    ws.fill_(0xff)
    for i, (size, rate) in enumerate([(300000, 0.9), (1000, 0.2), (2100000, 0.75), (5, 1.0), (300000, 0.9)]):
        x = _rand((size,), 20 + i, 2.0)
        y = kernels.prune(_dev(x, dev), rate, workspace=ws)
        assert bits_equal(to_np(y), oracle.prune(x, rate)), (size, rate)


@pytest.mark.parametrize("scale,zp,mode", [(0.3, 3.0, "HALF_AWAY_FROM_ZERO"), (0.0123, -7.0, "HALF_TO_EVEN"),
                                           (1.9999999, 0.0, "HALF_AWAY_FROM_ZERO"), (0.125, 1.0, "HALF_TO_EVEN"),
                                           (3e-39, 0.0, "HALF_AWAY_FROM_ZERO"), (1e30, 100.0, "HALF_AWAY_FROM_ZERO"),
                                           (-0.7, 5.0, "HALF_TO_EVEN")])
def test_quantize_linear_every_fp32_value(dev, scale, zp, mode):
    """All 2^32 bit patterns of x for a few scales (ordinary, all-ones significand, power of two, subnormal, huge,
    negative) against quantize_linear.cpp:78-111 restated with torch operations: an fp32 divide by a device operand,
    rounding in float64 (exact), fp32 add, clamp.  The kernel estimates most quotients with a reciprocal; this pins
    that no estimate changes an output."""
    import torch
    s = torch.tensor([scale], dtype=torch.float32, device=dev)
    z = torch.tensor([zp], dtype=torch.float32, device=dev)
    chunk = 1 << 27
    for start in range(0, 1 << 32, chunk):
        lo = start - (1 << 32) if start >= (1 << 31) else start
        x = torch.arange(lo, lo + chunk, dtype=torch.int32, device=dev).view(torch.float32)
        y = kernels.quantize_linear(x, s, z.clone(), round_mode=mode)
        q = (x / s).double()
        if mode == "HALF_TO_EVEN":
            t = torch.round(q)
        else:
            t = torch.copysign(torch.floor(q.abs() + 0.5), q)
        ref = torch.clamp(t.float() + z, -128.0, 127.0)
        same = (y == ref) | (torch.isnan(y) & torch.isnan(ref))
        if not bool(same.all()):
            i = int((~same).nonzero()[0])
            raise AssertionError("x=%r (bits %#x): got %r want %r" % (float(x[i]), start + i, float(y[i]), float(ref[i])))
