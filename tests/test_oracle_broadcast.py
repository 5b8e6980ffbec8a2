"""The oracle's restatement of two-input arithmetic with broadcasting (utils/base_transform_binary.hpp:58-336), pinned.

The restatement walks the reference's own index arithmetic (merged axis groups, strides that are 0 along a broadcast
group, one output index after the other).  What pins it: numpy's broadcasting, an independent implementation of the same
rule (forward bit for bit); for the gradients, sums over the broadcast axes -- exact on integer-valued data, where
every order of additions gives the same fp32 result (so a wrong index, a missing term or a swapped operand shows as a
different integer), and in float64 at rounding tolerance on real-valued data; the sequential fp32 order itself against
a plain Python loop on a small case.  The element-wise power's bits (std::pow) are not pinned: numpy's powf stands in.
"""
import numpy as np
import pytest

import oracle

SHAPES = [((3, 4, 5), (3, 4, 5)), ((3, 4, 5), (3, 1, 5)), ((3, 4, 5), (1, 4, 1)), ((1, 4, 1), (3, 4, 5)),
          ((2, 1, 3, 1, 2), (1, 4, 3, 5, 1)), ((6,), (1,)), ((1, 1), (7, 3)), ((2, 3, 1, 1), (2, 3, 4, 5)),
          ((4, 1, 1, 6), (4, 2, 3, 6)), ((), ())]
OPS = {"sub2": np.subtract, "mul2": np.multiply, "div2": np.divide, "add2": np.add}


def _data(shape, rng, ints=False, positive=False):
    if ints:
        v = rng.integers(-4, 5, size=shape).astype(np.float32)
        return np.where(v == 0, np.float32(1), v) if positive else v
    v = rng.standard_normal(shape).astype(np.float32)
    return (np.abs(v) + np.float32(0.5)) if positive else v


@pytest.mark.parametrize("s0,s1", SHAPES)
@pytest.mark.parametrize("op", sorted(OPS))
def test_forward_is_numpy_broadcasting(op, s0, s1):
    rng = np.random.default_rng(len(s0) * 10 + len(op))
    a, b = _data(s0, rng), _data(s1, rng, positive=(op == "div2"))
    y = oracle.transform_binary(op, a, b)
    with np.errstate(all="ignore"):
        ref = OPS[op](a, b).astype(np.float32)
    assert y.shape == ref.shape and np.array_equal(y.view(np.uint32), ref.view(np.uint32))


def _unbroadcast(t, shape):
    axes = tuple(i for i, n in enumerate(shape) if n == 1 and t.shape[i] != 1)
    return t.sum(axis=axes, keepdims=True) if axes else t


@pytest.mark.parametrize("s0,s1", SHAPES)
@pytest.mark.parametrize("op", ["sub2", "mul2", "add2"])
def test_gradients_on_integer_data_are_exact_sums_over_the_broadcast_axes(op, s0, s1):
    rng = np.random.default_rng(7)
    a, b = _data(s0, rng, ints=True), _data(s1, rng, ints=True)
    dy = _data(np.broadcast_shapes(s0, s1), rng, ints=True)
    t0 = {"sub2": dy, "mul2": dy * b, "add2": dy}[op] + np.zeros_like(a)
    t1 = {"sub2": -dy, "mul2": dy * a, "add2": dy}[op] + np.zeros_like(b)
    assert np.array_equal(oracle.transform_binary_backward(op, 0, dy, a, b), _unbroadcast(t0, s0))
    assert np.array_equal(oracle.transform_binary_backward(op, 1, dy, a, b), _unbroadcast(t1, s1))
    g = _data(s1, rng, ints=True)
    assert np.array_equal(oracle.transform_binary_backward(op, 1, dy, a, b, g=g), g + _unbroadcast(t1, s1))


@pytest.mark.parametrize("s0,s1", SHAPES)
def test_div2_and_pow2_gradients_against_float64(s0, s1):
    rng = np.random.default_rng(8)
    a, b = _data(s0, rng, positive=True), _data(s1, rng, positive=True)
    dy = _data(np.broadcast_shapes(s0, s1), rng)
    a64, b64, d64 = a.astype(np.float64), b.astype(np.float64), dy.astype(np.float64)
    for op, t0, t1 in (("div2", d64 / b64, -d64 * a64 / (b64 * b64)),
                       ("pow2", d64 * b64 * a64 ** (b64 - 1), d64 * np.log(a64) * a64 ** b64)):
        g0 = oracle.transform_binary_backward(op, 0, dy, a, b)
        g1 = oracle.transform_binary_backward(op, 1, dy, a, b)
        r0, r1 = _unbroadcast(t0 + np.zeros(s0), s0), _unbroadcast(t1 + np.zeros(s1), s1)
        assert np.allclose(g0, r0, rtol=2e-5, atol=2e-5) and np.allclose(g1, r1, rtol=2e-5, atol=2e-5)
    y = oracle.transform_binary("pow2", a, b)
    assert np.allclose(y, a64 ** b64, rtol=1e-6)


def test_the_sum_runs_in_ascending_output_index_in_fp32():
    """Values whose fp32 sum depends on the order: the restatement must give what the reference's loop gives
    (g[idx1] = g[idx1] + term, one output element after the other)."""
    a = np.ones((2, 3, 2), np.float32)
    b = np.ones((1, 3, 1), np.float32)
    dy = np.array([1e8, 1.0, 3.0, 1e-3, 2.0, 5.0, -1e8, 1.0, 1.0, 1e8, 1e-3, -1e8], np.float32).reshape(2, 3, 2)
    got = oracle.transform_binary_backward("add2", 1, dy, a, b)
    want = np.zeros(3, np.float32)
    for idx in range(12):
        c = (idx // 2) % 3
        want[c] = np.float32(want[c] + dy.reshape(-1)[idx])
    assert np.array_equal(got.reshape(-1), want)
    assert not np.array_equal(want, dy.astype(np.float64).sum((0, 2)).astype(np.float32))   # the order matters here


def test_errors():
    with pytest.raises(oracle.OracleError):
        oracle.transform_binary("add2", np.zeros((2, 3)), np.zeros((3,)))
    with pytest.raises(oracle.OracleError):
        oracle.transform_binary("add2", np.zeros((2, 3)), np.zeros((2, 2)))
