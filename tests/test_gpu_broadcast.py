"""Two-input arithmetic with broadcasting on the GPU (nbla_hip_broadcast2_f32 and its backward) against the oracle's
restatement of utils/base_transform_binary.hpp:58-336.

Bit-exact: the forward of sub2 / mul2 / div2 / add2 and the gradient of an operand that is not broadcast (one IEEE
operation per element, or the reference's expression operation by operation).  At rounding tolerance: the gradient of a
broadcast operand (the kernels add its terms as interleaved partial sums in a fixed order, the reference one after the
other) -- and
exact again on integer-valued data, where every order gives the same sum.  The element-wise power uses the device's
powf / logf: a few ulp from the host's, not pinned."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, to_np

pytestmark = pytest.mark.gpu

SHAPES = [((3, 4, 5), (3, 4, 5)), ((3, 4, 5), (3, 1, 5)), ((3, 4, 5), (1, 4, 1)), ((1, 4, 1), (3, 4, 5)),
          ((2, 1, 3, 1, 2), (1, 4, 3, 5, 1)), ((600,), (1,)), ((1, 1), (70, 33)), ((2, 3, 1, 1), (2, 3, 40, 50)),
          ((4, 1, 1, 6), (4, 20, 30, 6)), ((32, 64, 14, 14), (1, 64, 1, 1)), ((1, 2, 1, 2, 1, 2, 1, 2), (2, 1, 2, 1, 2, 1, 2, 1)),
          # the sums of a broadcast operand spread over blocks: a bias over the last axis, per channel, per sample, a
          # scalar against a long run (cut into pieces) and against a run no piece divides, kept groups on both sides
          # of a broadcast one, innermost extents that are (not) multiples of four
          ((4096, 300), (1, 300)), ((300, 4096), (300, 1)), ((16, 8, 56, 56), (1, 1, 1, 1)), ((1,), (100003,)),
          ((6, 40, 30, 56), (1, 40, 1, 56)), ((6, 40, 30, 56), (6, 1, 30, 1)), ((20, 50, 7, 3), (1, 50, 1, 1)),
          ((8, 16, 27, 27), (8, 1, 1, 1)), ((2, 3, 2000, 6), (1, 3, 1, 6))]


def _dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _data(shape, rng, positive=False, ints=False):
    if ints:
        return rng.integers(-4, 5, size=shape).astype(np.float32)
    v = rng.standard_normal(shape).astype(np.float32)
    return (np.abs(v) + np.float32(0.5)) if positive else v


def _abs_terms(op, i, dy, a, b, shape):
    """Per element of operand i, the sum of the magnitudes of its gradient terms (float64): what the rounding error of
    an fp32 sum, in whatever order, is relative to."""
    dy, a, b = dy.astype(np.float64), a.astype(np.float64), b.astype(np.float64)
    if op in ("sub2", "add2"):
        t = np.abs(dy)
    elif op == "mul2":
        t = np.abs(dy * (b if i == 0 else a))
    else:
        t = np.abs(dy / b) if i == 0 else np.abs(dy * a / (b * b))
    t = np.broadcast_to(t, dy.shape)
    axes = tuple(ax for ax in range(dy.ndim) if shape[ax] == 1 and dy.shape[ax] != 1)
    return t.sum(axis=axes, keepdims=True).reshape(shape) if axes else t.reshape(shape)


@pytest.mark.parametrize("s0,s1", SHAPES)
@pytest.mark.parametrize("op", ["sub2", "mul2", "div2", "add2"])
def test_forward_and_gradients(dev, op, s0, s1):
    rng = np.random.default_rng(3)
    a, b = _data(s0, rng), _data(s1, rng, positive=(op == "div2"))
    a.reshape(-1)[:1] = -0.0
    dy = _data(np.broadcast_shapes(s0, s1), rng)
    y = kernels.broadcast2(op, _dev(a, dev), _dev(b, dev))
    assert bits_equal(to_np(y), oracle.transform_binary(op, a, b))
    for i, shape in ((0, s0), (1, s1)):
        g = kernels.broadcast2_backward(op, i, _dev(dy, dev), _dev(a, dev), _dev(b, dev))
        ref = oracle.transform_binary_backward(op, i, dy, a, b)
        if tuple(shape) == tuple(dy.shape):
            assert bits_equal(to_np(g), ref)
        else:
            # (both sums are fp32, in different orders: they differ by rounding, relative to the sum of |terms|)
            tol = 2e-5 * max(1.0, float(np.abs(ref).max())) + 2e-7 * _abs_terms(op, i, dy, a, b, shape)
            assert (np.abs(to_np(g) - ref) <= tol).all()
        old = _data(shape, rng)
        g2 = kernels.broadcast2_backward(op, i, _dev(dy, dev), _dev(a, dev), _dev(b, dev), dx=_dev(old, dev))
        ref2 = oracle.transform_binary_backward(op, i, dy, a, b, g=old)
        if tuple(shape) == tuple(dy.shape):
            assert bits_equal(to_np(g2), ref2)
        else:
            tol = 2e-5 * max(1.0, float(np.abs(ref2).max())) + 2e-7 * _abs_terms(op, i, dy, a, b, shape)
            assert (np.abs(to_np(g2) - ref2) <= tol).all()
        again = kernels.broadcast2_backward(op, i, _dev(dy, dev), _dev(a, dev), _dev(b, dev))
        assert bits_equal(to_np(again), to_np(g))                       # the same from run to run


@pytest.mark.parametrize("s0,s1", SHAPES)
def test_reduced_gradients_are_exact_on_integer_data(dev, s0, s1):
    rng = np.random.default_rng(4)
    a, b = _data(s0, rng, ints=True), _data(s1, rng, ints=True)
    dy = _data(np.broadcast_shapes(s0, s1), rng, ints=True)
    for op in ("sub2", "mul2", "add2"):
        for i in (0, 1):
            g = kernels.broadcast2_backward(op, i, _dev(dy, dev), _dev(a, dev), _dev(b, dev))
            assert np.array_equal(to_np(g), oracle.transform_binary_backward(op, i, dy, a, b))


@pytest.mark.parametrize("s0,s1", SHAPES[:6])
def test_elementwise_power(dev, s0, s1):
    rng = np.random.default_rng(5)
    a, b = _data(s0, rng, positive=True), _data(s1, rng)
    dy = _data(np.broadcast_shapes(s0, s1), rng)
    y = to_np(kernels.broadcast2("pow2", _dev(a, dev), _dev(b, dev)))
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert np.allclose(y, a64 ** b64, rtol=2e-6)
    for i, t in ((0, dy * b64 * a64 ** (b64 - 1)), (1, dy * np.log(a64) * a64 ** b64)):
        g = to_np(kernels.broadcast2_backward("pow2", i, _dev(dy, dev), _dev(a, dev), _dev(b, dev)))
        ref = oracle.transform_binary_backward("pow2", i, dy, a, b)
        assert np.allclose(g, ref, rtol=3e-5, atol=3e-5)


def test_errors(dev):
    a, b = torch.zeros(2, 3, device=dev), torch.zeros(2, 2, device=dev)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.broadcast2("add2", a, b)
    assert ei.value.code == kernels.ERR_VALUE
