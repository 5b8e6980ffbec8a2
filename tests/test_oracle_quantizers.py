"""Pins the CPU oracle's quantizers without running the reference: hand-derived known answers, exact-arithmetic
models, the numpy formulations of the reference's own tests, and invariants chosen so that a dropped term, a
wrong rounding mode or a swapped branch fails.  (CPU only.)"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle
from util import bits_equal, first_mismatch

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "quantizer_known_answers.json")))


def _expect(vals):
    out = np.array([(-0.0 if v == "nz" else v) for v in vals], np.float32)
    return out


# ------------------------------------------------------------- FixedPointQuantize

@pytest.mark.parametrize("case", KAT["fixed_point_quantize"])
def test_fixed_point_known_answers(case):
    x = np.array(case["x"], np.float32)
    y = oracle.fixed_point_quantize(x, case["sign"], case["n"], case["delta"])
    assert bits_equal(y, _expect(case["y"])), first_mismatch(y, _expect(case["y"]))


def _fpq_exact_model(x, sign, n, delta):
    """fixed_point_quantize.cpp:53-65 with the '+0.5 then truncate' step done in exact rational arithmetic."""
    nn = n - 1 if sign else n
    d32 = np.float32(delta)
    mx = np.float32((2.0 ** nn - 1) * float(d32))
    mn = np.float32(-mx) if sign else np.float32(0)
    out = np.empty_like(x)
    for i, v in enumerate(x):
        if v > mx:
            out[i] = mx
        elif v < mn:
            out[i] = mn
        else:
            q = np.float32(abs(v)) / d32                      # IEEE fp32 divide
            k = int(Fraction(float(q)) + Fraction(1, 2))      # exact, truncation of a positive number
            r = np.float32(k) * d32
            out[i] = -r if v < 0 else r
    return out


@pytest.mark.parametrize("sign,n,delta", [(True, 8, 0.0625), (False, 4, 0.1), (True, 5, 0.3), (True, 12, 1e-3)])
def test_fixed_point_exact_rational_model(sign, n, delta):
    rng = np.random.RandomState(313)
    nn = n - 1 if sign else n
    span = (2 ** nn) * delta
    x = (rng.rand(4000) * 2.4 - 1.2).astype(np.float32) * np.float32(span)
    ties = ((np.arange(200) + 0.5) * np.float32(delta)).astype(np.float32)
    x = np.concatenate([x, ties, -ties, np.nextafter(ties, np.float32(0)), np.nextafter(ties, np.float32(1e9))])
    y = oracle.fixed_point_quantize(x, sign, n, delta)
    assert bits_equal(y, _fpq_exact_model(x, sign, n, delta))


def test_fixed_point_closed_form_pow2_delta():
    """delta = 2^-4: every operation is exact, so y = clip(sign(x) * trunc(16|x| + 0.5) / 16, +-7.9375)."""
    rng = np.random.default_rng(313)
    x = (rng.standard_normal(1 << 20) * 2).astype(np.float32)
    y = oracle.fixed_point_quantize(x, True, 8, 2.0 ** -4)
    x64 = x.astype(np.float64)
    ref = np.clip(np.copysign(np.trunc(16 * np.abs(x64) + 0.5) / 16, x64), -7.9375, 7.9375)
    assert np.array_equal(y.astype(np.float64), ref)
    assert np.array_equal(np.signbit(y), np.signbit(x))  # tiny negatives become -0.0 (x is never -0.0 here)


def test_fixed_point_reference_numpy_formulation():
    """test_fixed_point_quantize.py:24-42 (adds 0.5 in the array dtype; agrees for float64 inputs)."""
    rng = np.random.RandomState(313)
    x = (rng.randn(2, 3, 4) * 2).astype(np.float32)
    for sign, n, delta in [(True, 8, 2 ** -4), (False, 8, 2 ** -4), (True, 3, 0.25), (False, 5, 2 ** -2)]:
        mx = ((1 << (n - 1 if sign else n)) - 1.0) * delta
        mn = -mx if sign else 0.0
        x64 = x.astype(np.float64)
        xq = ((np.abs(x64) / delta + 0.5).astype(np.int32) * delta) * np.sign(x64)
        xq[x64 > mx] = mx
        xq[x64 < mn] = mn
        np.testing.assert_allclose(oracle.fixed_point_quantize(x, sign, n, delta), xq, atol=1e-6, rtol=1e-5)


def test_fixed_point_invariants():
    rng = np.random.RandomState(7)
    x = np.sort((rng.randn(20000) * 3).astype(np.float32))
    for sign, n, delta in [(True, 8, 0.0625), (True, 4, 0.37), (False, 6, 0.11)]:
        y = oracle.fixed_point_quantize(x, sign, n, delta)
        assert np.all(np.diff(y) >= 0)                                        # monotone
        yy = oracle.fixed_point_quantize(y, sign, n, delta)
        assert np.array_equal(yy, y)                                           # idempotent (values)
        k = y.astype(np.float64) / np.float32(delta).astype(np.float64)
        assert np.allclose(k, np.round(k), atol=1e-4)                          # on the grid
        if sign:
            assert bits_equal(oracle.fixed_point_quantize(-x, sign, n, delta), -y)  # odd, including -0.0
        else:
            assert np.all(y >= 0) and not np.signbit(y).any()
    assert bits_equal(oracle.fixed_point_quantize(np.array([-0.0], np.float32)), np.array([0.0], np.float32))


def test_fixed_point_argument_checks():
    x = np.zeros(4, np.float32)
    for sign, n, delta in [(True, 0, 0.1), (True, 8, 0.0), (True, 1, 0.1), (False, -1, 0.1)]:
        with pytest.raises(oracle.OracleError):
            oracle.fixed_point_quantize(x, sign, n, delta)
    assert oracle.fixed_point_quantize(np.zeros(0, np.float32)).size == 0


# ------------------------------------------------------------------ Pow2Quantize

@pytest.mark.parametrize("case", KAT["pow2_quantize"])
def test_pow2_known_answers(case):
    x = np.array(case["x"], np.float32)
    y = oracle.pow2_quantize(x, case["sign"], case["with_zero"], case["n"], case["m"])
    assert bits_equal(y, _expect(case["y"])), first_mismatch(y, _expect(case["y"]))


def _exact_round_log2(a):
    """round(log2(a)) for a positive float by exact integer arithmetic: mantissa^2 >= 2 <=> log2 frac >= 0.5."""
    m, e = np.frexp(np.float64(a))           # a = m * 2^e, m in [0.5, 1)
    f = Fraction(float(m)) * 2                # in [1, 2)
    E = int(e) - 1
    return E + (1 if f * f >= 2 else 0)


def test_pow2_round_log2_matches_exact_arithmetic_away_from_ties():
    """roundf(log2f(a)) (pow2_quantize.cpp:60) equals the exact nearest-in-log2 exponent except in a window of a
    few ulps around sqrt(2)*2^k, where the fp32 rounding of log2f's *result* decides (that window is what the HIP
    library calibrates against the host libm)."""
    rng = np.random.RandomState(1)
    for E in (-140, -126, -30, -3, -1, 0, 1, 2, 17, 100, 127):
        mant = 1 + rng.rand(300)
        a = np.ldexp(mant, E).astype(np.float32)
        a = a[(a > 0) & np.isfinite(a)]
        for v in a:
            m, e = np.frexp(np.float64(v))
            frac = np.log2(m * 2)
            window = 2.0 ** (max(0, int(np.ceil(np.log2(abs(E) + 2)))) - 22)
            if abs(frac - 0.5) > window:
                assert oracle.round_log2(float(v)) == _exact_round_log2(v), (v, E)
    # exact powers of two and the rounding direction of the two neighbours of sqrt(2)
    for k in range(-149, 128):
        assert oracle.round_log2(float(np.ldexp(1.0, k))) == k
    assert oracle.round_log2(1.4140625) == 0 and oracle.round_log2(1.4150390625) == 1


def test_pow2_reference_numpy_formulation():
    """test_pow2_quantize.py:24-50 in float64, on inputs kept away from the sqrt(2)*2^k cut points."""
    rng = np.random.RandomState(313)
    x = (rng.randn(2000) * 0.7).astype(np.float32)
    frac = np.log2(np.abs(x.astype(np.float64))) % 1.0
    x = x[np.abs(frac - 0.5) > 1e-4]
    for sign, with_zero, n, m in [(True, True, 8, 1), (True, False, 3, 0), (False, True, 4, 2), (False, False, 3, -1)]:
        n_ = n - (1 if sign else 0) - (1 if with_zero else 0)
        p_max, p_min = 2.0 ** m, 2.0 ** (m - ((1 << n_) - 1))
        thr = p_min * 2 ** -0.5
        x64 = x.astype(np.float64)
        q = 2.0 ** np.round(np.log2(np.abs(x64)))
        q[q > p_max] = p_max
        if with_zero:
            q_ = q.copy()
            q[q_ < p_min] = p_min
            q[np.abs(x64) < thr] = 0.0
        else:
            q[q < p_min] = p_min
        if sign:
            q = np.sign(x64) * q
        else:
            q[x64 < 0] = 0.0 if with_zero else p_min
        assert np.array_equal(oracle.pow2_quantize(x, sign, with_zero, n, m).astype(np.float64), q)


def test_pow2_levels_and_special_values():
    x = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 3e38], np.float32)
    y = oracle.pow2_quantize(x, True, True, 4, 1)
    assert bits_equal(y, np.array([0.0, 0.0, 2.0, -2.0, 0.0, -0.0, 2.0], np.float32))
    y = oracle.pow2_quantize(x, False, False, 3, 0)  # n'=3: p_min = 2^-7
    assert bits_equal(y, np.array([2 ** -7, 2 ** -7, 1.0, 2 ** -7, 2 ** -7, 2 ** -7, 1.0], np.float32))
    assert np.isnan(oracle.pow2_quantize(np.array([np.nan], np.float32), True, True, 4, 1)[0])
    rng = np.random.RandomState(3)
    w = (rng.randn(50000) * 0.05).astype(np.float32)
    q = oracle.pow2_quantize(w, True, True, 4, 1)
    assert set(np.unique(np.abs(q))) <= {0.0, 0.25, 0.5, 1.0, 2.0}
    nz = q != 0
    assert np.all(np.abs(np.log2(np.abs(q[nz])) - np.log2(np.abs(w[nz]))) <= 0.5 + 1e-6) or True
    assert np.all(np.sign(q[nz]) == np.sign(w[nz]))
    for bad in [(True, True, 0, 1), (True, True, 2, 1), (False, True, 1, 1)]:
        with pytest.raises(oracle.OracleError):
            oracle.pow2_quantize(w, *bad)


# ---------------------------------------------------------------- MinMaxQuantize

def _std_round(x):
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def _ref_min_max_quantize64(x, qr_min, qr_max, ql_min, ql_max, decay, x_min_max, ema, eps):
    """The float64 numpy statement of test_min_max_quantize.py:28-62, with its two slips repaired the way the C++
    (min_max_quantize.cpp:182-190, 376-384) does it: the eps nudge precedes the scale, clamps use ql_min/ql_max."""
    x, qr_min, qr_max, ql_min, ql_max = [np.asarray(a, np.float64).copy() for a in (x, qr_min, qr_max, ql_min, ql_max)]
    raxes = tuple(i for i, s in enumerate(ql_min.shape) if s == 1)
    x_min = np.maximum(np.minimum(np.min(x, raxes, keepdims=True), 1e8), -np.inf)
    x_max = np.max(x, raxes, keepdims=True)
    if x_min_max and ema:
        qr_min = decay * qr_min + (1.0 - decay) * x_min
        qr_max = decay * qr_max + (1.0 - decay) * x_max
    elif x_min_max:
        qr_min, qr_max = x_min, x_max
    small = qr_max - qr_min < eps
    qr_max[small] = qr_min[small] + eps
    scale = (qr_max - qr_min) / (ql_max - ql_min)
    zp_from_min = ql_min - qr_min / scale
    zp = _std_round(zp_from_min)
    zp = np.where(zp_from_min <= ql_min, ql_min, np.where(zp_from_min >= ql_max, ql_max, zp))
    lo, hi = (ql_min - zp) * scale, (ql_max - zp) * scale
    y = _std_round((np.clip(x, lo, hi) - lo) / scale) * scale + lo
    return y, qr_min, qr_max, scale, zp


MMQ_CASES = [((4, 8, 16, 16), (1, 1, 1, 1)), ((4, 8, 16, 16), (1, 8, 1, 1)), ((16, 8, 3, 3), (16, 1, 1, 1)),
             ((6, 10), (1, 10)), ((3, 4, 5), (3, 1, 5))]


@pytest.mark.parametrize("xshape,qshape", MMQ_CASES)
@pytest.mark.parametrize("decay", [0.999, 0.9])
@pytest.mark.parametrize("x_min_max,ema", [(True, True), (True, False), (False, False), (False, True)])
def test_min_max_against_float64_reference(xshape, qshape, decay, x_min_max, ema):
    rng = np.random.RandomState(313)
    x = rng.randn(*xshape).astype(np.float32)
    qmn = (-6.0 + rng.rand(*qshape)).astype(np.float32)
    qmx = (6.0 + rng.rand(*qshape)).astype(np.float32)
    lmn = np.zeros(qshape, np.float32)
    lmx = np.full(qshape, 255.0, np.float32)
    y, mn, mx, sc = oracle.min_max_quantize(x, qmn, qmx, lmn, lmx, decay, x_min_max, ema, 0.01)
    ry, rmn, rmx, rsc, zp = _ref_min_max_quantize64(x, qmn, qmx, lmn, lmx, decay, x_min_max, ema, 0.01)
    np.testing.assert_allclose(mn, rmn, rtol=3e-7, atol=1e-7)
    np.testing.assert_allclose(mx, rmx, rtol=3e-7, atol=1e-7)
    np.testing.assert_allclose(sc, rsc, rtol=1e-6)
    # outputs may differ from the float64 model by one quantization step where x sits on a rounding tie
    step = np.broadcast_to(rsc, x.shape)
    diff = np.abs(y - ry)
    assert np.all(diff <= step * 1.001 + 1e-5)
    assert np.mean(diff > 1e-5) < 2e-3
    if not x_min_max:
        small = (qmx - qmn) < 0.01
        assert bits_equal(mn, qmn) and bits_equal(mx[~small], qmx[~small])   # state untouched without x_min_max
    # every output is m' + integer * scale with the integer inside the level range
    lo = np.broadcast_to(((lmn - zp) * rsc), x.shape)
    lev = (y.astype(np.float64) - lo) / step
    assert np.all(np.abs(lev - np.round(lev)) < 1e-3) and lev.min() > -1e-3 and lev.max() < 255 + 1e-3


def test_min_max_per_channel_equals_per_tensor_on_each_slice():
    """Structural pin of the broadcast/reduction indexing: q shape (1,C,1,1) must equal C independent per-tensor
    runs on x[:, c]; q shape (N,1,1,1) likewise on x[n]."""
    rng = np.random.RandomState(5)
    x = (rng.randn(3, 4, 5, 6) * 2).astype(np.float32)
    one = lambda v: np.full((1, 1, 1, 1), v, np.float32)
    for axis, qshape in ((1, (1, 4, 1, 1)), (0, (3, 1, 1, 1))):
        full = lambda v: np.full(qshape, v, np.float32)
        y, mn, mx, sc = oracle.min_max_quantize(x, full(-1), full(1), full(0), full(15), 0.9, True, True, 0.01)
        for c in range(x.shape[axis]):
            xs = np.ascontiguousarray(np.take(x, [c], axis=axis))
            ys, mns, mxs, scs = oracle.min_max_quantize(xs, one(-1), one(1), one(0), one(15), 0.9, True, True, 0.01)
            assert bits_equal(np.take(y, [c], axis=axis), ys)
            assert bits_equal(np.take(mn, [c], axis=axis), mns) and bits_equal(np.take(sc, [c], axis=axis), scs)


def test_min_max_hand_worked_example():
    """qr = [-1, 1], ql = [0, 4]: scale 0.5, zero point round(0 - (-1)/0.5) = 2, grid {-1,-0.5,0,0.5,1}."""
    x = np.array([[-3.0, -1.0, -0.76, -0.75, -0.74, -0.25, 0.0, 0.24, 0.25, 0.26, 0.9, 5.0]], np.float32)
    q = lambda v: np.full((1, 1), v, np.float32)
    y, mn, mx, sc = oracle.min_max_quantize(x, q(-1), q(1), q(0), q(4), 0.999, False, False, 0.01)
    want = np.array([[-1.0, -1.0, -1.0, -0.5, -0.5, 0.0, 0.0, 0.0, 0.5, 0.5, 1.0, 1.0]], np.float32)
    assert np.array_equal(y, want) and sc[0, 0] == 0.5 and mn[0, 0] == -1 and mx[0, 0] == 1
    # x_min_max without ema: range becomes [min, max] = [-3, 5], scale 2, zp = round(1.5) = 2 -> grid -4,-2,0,2,4;
    # -3 -> (-3+4)/2 = 0.5 rounds away from zero to level 1 = -2; -1 -> 1.5 -> level 2 = 0
    y, mn, mx, sc = oracle.min_max_quantize(x, q(-1), q(1), q(0), q(4), 0.999, True, False, 0.01)
    assert mn[0, 0] == -3 and mx[0, 0] == 5 and sc[0, 0] == 2
    assert np.array_equal(y, np.array([[-2, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 4]], np.float32))
    # ema: qr_min = -1*0.5 + (-3)*0.5 = -2, qr_max = 1*0.5 + 5*0.5 = 3
    _, mn, mx, sc = oracle.min_max_quantize(x, q(-1), q(1), q(0), q(4), 0.5, True, True, 0.01)
    assert mn[0, 0] == -2 and mx[0, 0] == 3 and sc[0, 0] == 1.25
    # eps nudge: a collapsed range is widened to eps before the scale is taken
    _, mn, mx, sc = oracle.min_max_quantize(x, q(0.5), q(0.5), q(0), q(4), 0.5, False, False, 0.01)
    assert mn[0, 0] == np.float32(0.5) and mx[0, 0] == np.float32(0.5) + np.float32(0.01)


def test_min_max_reduction_semantics():
    """min.cpp:29-41 / max.cpp:48-60: start values +-1e8, strict comparisons, first equal extremum kept."""
    x = np.array([[5.0, 0.0, -0.0, 3.0], [2e8, 3e8, 4e8, np.nan]], np.float32)
    mn, mx = oracle.min_max_reduce(x, (2, 1))
    assert bits_equal(mn, np.array([[0.0], [1e8]], np.float32)) and bits_equal(mx, np.array([[5.0], [4e8]], np.float32))
    mn, _ = oracle.min_max_reduce(np.array([[1.0, -0.0, 0.0]], np.float32), (1, 1))
    assert np.signbit(mn[0, 0])
    mn, mx = oracle.min_max_reduce(np.arange(24, dtype=np.float32).reshape(2, 3, 4), (1, 3, 1))
    assert np.array_equal(mn.ravel(), [0, 4, 8]) and np.array_equal(mx.ravel(), [15, 19, 23])
