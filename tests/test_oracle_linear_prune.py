"""Pins of the oracle's QuantizeLinear / DequantizeLinear / Prune restatements (CPU only): numpy's own rounding
routines (rint = half-to-even, floor(|t| + 0.5) = half-away), known answers at the ties and range ends, the
in-place treatment of the zero point, and Prune against a numpy order statistic."""
import numpy as np
import pytest

import oracle


def _rand(shape, seed, scale=1.0):
    return (np.random.RandomState(seed).randn(*shape) * scale).astype(np.float32)


def _ref_quantize(x, scale, zp, mode, lo, hi):
    t = (x / scale).astype(np.float32)                         # one fp32 division
    if mode == "HALF_TO_EVEN":
        r = np.rint(t)
        z = np.rint(zp)
    else:
        r = np.sign(t) * np.floor(np.abs(t.astype(np.float64)) + 0.5)
        z = np.sign(zp) * np.floor(np.abs(zp.astype(np.float64)) + 0.5)
    z = np.clip(z, lo, hi).astype(np.float32)
    return np.clip((r.astype(np.float32) + z).astype(np.float32), lo, hi), z


@pytest.mark.parametrize("mode", ["HALF_AWAY_FROM_ZERO", "HALF_TO_EVEN"])
@pytest.mark.parametrize("narrow,dtype,lo,hi", [(False, 1, -128, 127), (True, 1, -127, 127), (False, 2, 0, 255),
                                                (True, 2, 1, 255)])
@pytest.mark.parametrize("sshape,zshape", [((1, 1, 1), (1, 1, 1)), ((1, 5, 1), (1, 5, 1)), ((3, 1, 1), (1, 1, 7)),
                                           ((3, 5, 7), (1, 5, 1))])
def test_quantize_linear_against_numpy_rounding(mode, narrow, dtype, lo, hi, sshape, zshape):
    x = _rand((3, 5, 7), 1, 40.0)
    x.ravel()[:8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 1e4, -1e4]
    scale = (np.abs(_rand(sshape, 2)) + 0.25).astype(np.float32)
    if sshape == (1, 1, 1):
        scale[...] = 1.0                                        # keeps the planted ties exact
    zp = _rand(zshape, 3, 30.0)
    zp.ravel()[0] = 2.5
    y, zp_out = oracle.quantize_linear(x, scale, zp, mode, narrow, dtype)
    ref, zref = _ref_quantize(x, scale, zp, mode, lo, hi)
    assert np.array_equal(zp_out, zref)
    assert np.array_equal(y, ref)
    assert y.min() >= lo and y.max() <= hi and np.array_equal(y, np.rint(y))


def test_quantize_linear_known_answers():
    one = np.float32([[1.0]])
    x = np.float32([[0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, -128.5, -129.5, 0.49999997]])
    y, _ = oracle.quantize_linear(x, one, np.float32([[0.0]]), "HALF_AWAY_FROM_ZERO")
    assert y.tolist() == [[1, 2, 3, -1, -2, 127, 127, -128, -128, 0]]
    y, _ = oracle.quantize_linear(x, one, np.float32([[0.0]]), "HALF_TO_EVEN")
    assert y.tolist() == [[0, 2, 2, 0, -2, 126, 127, -128, -128, 0]]
    # the zero point is rounded, saturated and written back before it is added
    y, zp = oracle.quantize_linear(np.float32([[1.0, -1.0]]), one, np.float32([[300.4]]), dtype=2)
    assert zp.tolist() == [[255.0]] and y.tolist() == [[255.0, 254.0]]
    with pytest.raises(oracle.OracleError):
        oracle.quantize_linear(x, one, np.float32([[0.0]]), dtype=5)
    with pytest.raises(oracle.OracleError):
        oracle.quantize_linear(np.zeros((2, 3), np.float32), np.ones((2, 2), np.float32), np.zeros((1, 1), np.float32))


@pytest.mark.parametrize("sshape,zshape", [((1, 1), (1, 1)), ((1, 6), (1, 6)), ((4, 1), (1, 6)), ((4, 6), (4, 6))])
def test_dequantize_linear_and_backward(sshape, zshape):
    x = np.rint(_rand((4, 6), 4, 50.0)).astype(np.float32)
    scale = (np.abs(_rand(sshape, 5)) + 0.1).astype(np.float32)
    zp = np.rint(_rand(zshape, 6, 5.0)).astype(np.float32)
    assert np.array_equal(oracle.dequantize_linear(x, scale, zp), ((x - zp).astype(np.float32) * scale))
    dy, old = _rand((4, 6), 7), _rand((4, 6), 8)
    assert np.array_equal(oracle.linear_quantize_backward(dy, scale, True), dy * scale)
    assert np.array_equal(oracle.linear_quantize_backward(dy, scale, True, dx=old), old + dy * scale)
    assert np.array_equal(oracle.linear_quantize_backward(dy, scale, False), dy / scale)
    assert np.array_equal(oracle.linear_quantize_backward(dy, scale, False, dx=old), old + dy / scale)


@pytest.mark.parametrize("size,rate", [(1, 0.5), (10, 0.0), (10, 1.0), (1000, 0.9), (4097, 0.33), (100000, 0.5)])
def test_prune_against_order_statistic(size, rate):
    x = _rand((size,), 9)
    if size > 3:
        x[::7] = x[3]                                           # ties at one magnitude, both signs
        x[::14] = -x[3]
    idx = int(np.float32(size - 1) * np.float32(rate))
    thresh = np.sort(np.abs(x))[idx] + (1.0 if rate == 1.0 else 0.0)
    y = oracle.prune(x, rate)
    assert np.array_equal(y, np.where(np.abs(x) < np.float32(thresh), np.float32(0), x))
    if rate == 1.0:
        assert not y.any() or np.abs(x).max() >= thresh
    if rate == 0.0:
        assert np.array_equal(y, x)


def test_prune_index_is_computed_in_float():
    """(x_size - 1) * rate is an int times a float: above 2^24 elements the product rounds."""
    size, rate = (1 << 24) + 3, np.float32(0.75)
    assert int(np.float32(size - 1) * rate) != int((size - 1) * 0.75)
    x = np.arange(size, dtype=np.float32)                       # |x| sorted: the threshold is the index itself
    y = oracle.prune(x, float(rate))
    kept = np.flatnonzero(y)
    assert kept[0] == int(np.float32(size - 1) * rate) or x[kept[0]] == np.float32(int(np.float32(size - 1) * rate))
    with pytest.raises(oracle.OracleError):
        oracle.prune(x[:4], 1.5)
