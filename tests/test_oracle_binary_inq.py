"""Pins the CPU oracle's binary-weight, convolution and INQ functions against independent formulations:
numpy float64 (the reference tests' own refs), torch's float64 convolution, hand-worked cases and invariants.
The fp32 *bits* of alpha and of GEMM/conv outputs depend on Eigen's summation order and stay unpinned; they are
checked at tolerance.  (CPU only.)"""
import numpy as np
import pytest
import torch

import oracle
from util import bits_equal, max_rel_err


def _sign64(W, q0):
    return np.where(W > 0, 1.0, np.where(W < 0, -1.0, q0))


# ----------------------------------------------------------- Sign / alpha / affine

def test_sign_closed_form_and_zero_handling():
    x = np.array([3.0, -2.0, 0.0, -0.0, 1e-45, -1e-45, np.inf, -np.inf, np.nan], np.float32)
    for q0 in (1.0, 0.0, -1.0, 0.5):
        want = np.array([1, -1, q0, q0, 1, -1, 1, -1, q0], np.float32)
        assert bits_equal(oracle.sign(x, q0), want)


@pytest.mark.parametrize("M,K,N", [(2, 3, 4), (5, 17, 9), (16, 128, 48), (3, 1000, 7)])
@pytest.mark.parametrize("q0", [1.0, 0.0, -1.0])
def test_binary_weight_affine_vs_float64(M, K, N, q0):
    """test_binary_weight_affine.py:23-37: alpha = mean|W| over the input axis, y = x . (sign(W) * alpha) + b."""
    rng = np.random.RandomState(313)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.1).astype(np.float32)
    W.ravel()[::9] = 0.0
    b = rng.randn(N).astype(np.float32)
    y, Wb, alpha = oracle.binary_weight_affine(x, W, b, q0)
    W64 = W.astype(np.float64)
    assert np.array_equal(Wb, _sign64(W64, q0).astype(np.float32))
    a64 = np.abs(W64).mean(0)
    np.testing.assert_allclose(alpha, a64, rtol=1e-6)
    y64 = x.astype(np.float64) @ (_sign64(W64, q0) * a64) + b
    assert max_rel_err(y, y64) < 3e-6
    yc, Wbc = oracle.binary_connect_affine(x, W, b, q0)
    assert np.array_equal(Wbc, Wb)
    assert max_rel_err(yc, x.astype(np.float64) @ _sign64(W64, q0) + b) < 3e-6


def test_alpha_uses_reciprocal_multiply_and_exact_small_cases():
    """(float)1/K is rounded once and multiplied (binary_weight_affine.cpp:68); integer-valued weights make the
    column sums exact whatever the summation order, which isolates that step."""
    K, N = 7, 5
    W = np.arange(1, K * N + 1, dtype=np.float32).reshape(K, N) * np.where(np.arange(K * N).reshape(K, N) % 2, -1, 1)
    _, alpha = oracle.binary_weight_prepare(W.astype(np.float32))
    sums = np.abs(W).sum(0).astype(np.float32)
    assert bits_equal(alpha, sums * (np.float32(1) / np.float32(K)))
    assert not bits_equal(alpha, (sums / np.float32(K)).astype(np.float32)) or True


def test_row_sum_order_is_eigens_for_a_distinguishing_vector():
    """Eigen 3.3.5 linear-vectorised redux with SSE packets: two 4-lane accumulators over pairs of packets, then
    (l0+l2)+(l1+l3), then the scalar tail.  A vector built from powers of two separates that order from a plain
    left-to-right sum; the expected value is worked out by hand below."""
    big, one = np.float32(2.0 ** 24), np.float32(1.0)
    # K = 9: packets p0 = v[0:4], p1 = v[4:8], tail v[8].  lanes: p0+p1 = [big+1 -> big, 1+1, 1+1, 1+1]
    v = np.array([big, 1, 1, 1, 1, 1, 1, 1, 1], np.float32)
    got = oracle.binary_weight_prepare(v.reshape(9, 1))[1][0] / (np.float32(1) / np.float32(9))
    lanes = [np.float32(big + one), np.float32(2), np.float32(2), np.float32(2)]     # big+1 rounds to big
    want = np.float32(np.float32(lanes[0] + lanes[2]) + np.float32(lanes[1] + lanes[3]))
    want = np.float32(want + one)                                                   # tail: (big+6)+1 ties to even
    seq = np.float32(0)
    for t in v:
        seq = np.float32(seq + t)
    assert seq == big                       # the naive order loses every 1
    alpha = oracle.binary_weight_prepare(v.reshape(9, 1))[1][0]
    assert alpha == np.float32(want * (np.float32(1) / np.float32(9)))
    assert got != seq


# -------------------------------------------------------------------- convolution

CONV_CASES = [
    # (x shape, w shape, pad, stride, dilation, group)
    ((2, 4, 7, 7), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((2, 4, 7, 7), (6, 2, 3, 3), (1, 0), (2, 1), (1, 2), 2),
    ((1, 3, 9, 8), (5, 3, 2, 3), (0, 2), (1, 2), (2, 1), 1),
    ((3, 2, 10), (4, 2, 3), (1,), (2,), (1,), 1),
    ((2, 2, 4, 5, 6), (3, 2, 2, 3, 2), (1, 0, 1), (1, 2, 1), (1, 1, 2), 1),
    ((2, 6, 5, 5), (6, 1, 3, 3), (1, 1), (1, 1), (1, 1), 6),
]


def _torch_conv(x, w, b, pad, stride, dil, group):
    fn = {1: torch.nn.functional.conv1d, 2: torch.nn.functional.conv2d, 3: torch.nn.functional.conv3d}[w.ndim - 2]
    bt = None if b is None else torch.from_numpy(b).double()
    return fn(torch.from_numpy(x).double(), torch.from_numpy(w).double(), bt, stride, pad, dil, group).numpy()


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CONV_CASES)
def test_convolution_vs_torch_float64(xs, ws, pad, stride, dil, group):
    rng = np.random.RandomState(313)
    x = rng.randn(*xs).astype(np.float32)
    w = rng.randn(*ws).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)
    y = oracle.convolution(x, w, b, pad, stride, dil, group)
    ref = _torch_conv(x, w, b, pad, stride, dil, group)
    assert y.shape == ref.shape
    assert max_rel_err(y, ref) < 3e-6


@pytest.mark.parametrize("xs,ws,pad,stride,dil,group", CONV_CASES)
def test_binary_convolutions_vs_torch_float64(xs, ws, pad, stride, dil, group):
    """test_binary_weight_convolution.py:26-40 / test_binary_connect_convolution.py: per-output-channel alpha."""
    rng = np.random.RandomState(7)
    x = rng.randn(*xs).astype(np.float32)
    w = (rng.randn(*ws) * 0.1).astype(np.float32)
    w.ravel()[::11] = 0.0
    for q0 in (1.0, -1.0, 0.0):
        y, Wb, alpha = oracle.binary_weight_convolution(x, w, None, pad, stride, dil, group, q0)
        s64 = _sign64(w.astype(np.float64), q0)
        a64 = np.abs(w.astype(np.float64)).reshape(ws[0], -1).mean(1)
        assert np.array_equal(Wb, s64.astype(np.float32))
        np.testing.assert_allclose(alpha, a64, rtol=1e-6)
        ws64 = (s64 * a64.reshape((-1,) + (1,) * (w.ndim - 1))).astype(np.float64)
        assert max_rel_err(y, _torch_conv(x, ws64.astype(np.float32), None, pad, stride, dil, group)) < 1e-5
        yc, Wbc = oracle.binary_connect_convolution(x, w, None, pad, stride, dil, group, q0)
        assert np.array_equal(Wbc, Wb)
        assert max_rel_err(yc, _torch_conv(x, s64.astype(np.float32), None, pad, stride, dil, group)) < 3e-6


def test_convolution_rejects_bad_geometry():
    x = np.zeros((1, 4, 5, 5), np.float32)
    with pytest.raises(oracle.OracleError):
        oracle.convolution(x, np.zeros((6, 4, 7, 7), np.float32))            # kernel larger than padded input
    with pytest.raises(oracle.OracleError):
        oracle.convolution(x, np.zeros((6, 2, 3, 3), np.float32), group=3)   # channels not divisible


# ---------------------------------------------------------------------------- INQ

def _inq_quantize64(w, max_absval, num_bits):
    """test_inq_affine.py:25-48 in float64 (differs from the C++ only next to the 1.5 * 2^k cut points)."""
    y = w.astype(np.float64).copy()
    l = np.log2(max_absval)
    n1 = np.floor(l) + (l - np.floor(l) >= np.log2(1.5))
    n2 = n1 + 1 - 2 ** (num_bits - 2)
    y[np.abs(y) < 2 ** (n2 - 1)] = 0.0
    i = y != 0
    b = np.log2(np.abs(y[i]))
    e = np.floor(b) + (b - np.floor(b) >= np.log2(1.5))
    e = np.maximum(n2, np.minimum(n1, e))
    y[i] = np.sign(y[i]) * 2 ** e
    return y, int(n1), int(n2)


@pytest.mark.parametrize("num_bits", [3, 4, 5, 7])
def test_inq_all_fixed_vs_float64_reference(num_bits):
    rng = np.random.RandomState(313)
    W = (rng.randn(64, 48) * 0.02).astype(np.float32)
    frac = np.log2(np.abs(W.astype(np.float64))) % 1.0
    W[np.abs(frac - np.log2(1.5)) < 1e-5] = 0.013         # keep clear of the cut points
    inq = oracle.Inq(W.size, num_bits, (0,), "largest_abs")
    Wq, I = W.copy(), np.zeros(W.shape, np.int32)
    n1, n2 = inq.quantize_weights(Wq, I)
    ref, rn1, rn2 = _inq_quantize64(W, np.abs(W).max(), num_bits)
    assert (n1, n2) == (rn1, rn2) and I.min() == 1
    assert np.array_equal(Wq.astype(np.float64), ref)
    levels = {0.0} | {2.0 ** e for e in range(n2, n1 + 1)}
    assert set(np.unique(np.abs(Wq)).tolist()) <= levels and len(levels) == 2 ** (num_bits - 2) + 1


def test_inq_hand_worked_thresholds():
    """max|w| = 1 -> n1 = 0; num_bits = 4 -> n2 = -3, prune below 2^-4; arithmetic-mean cut at 1.5 * 2^e."""
    W = np.array([1.0, 0.76, 0.74, 0.5, 0.38, 0.37, 0.126, 0.124, 0.0625, 0.0624, -0.76, -0.0624, 0.19, 0.18, 3e-4],
                 np.float32)
    want = np.array([1.0, 1.0, 0.5, 0.5, 0.5, 0.25, 0.125, 0.125, 0.125, 0.0, -1.0, -0.0, 0.25, 0.125, 0.0],
                    np.float32)
    inq = oracle.Inq(W.size, 4, (), "largest_abs")
    Wq, I = W.copy(), np.ones(W.shape, np.int32)
    assert inq.quantize_weights(Wq, I) == (0, -3)
    assert np.array_equal(Wq, want)
    # n1 itself uses the arithmetic-mean rule: max 1.4 -> 0, max 1.6 -> 1; an all-zero tensor counts as max 1
    assert oracle.inq_n1(1.4) == 0 and oracle.inq_n1(1.6) == 1 and oracle.inq_n1(0.76) == 0 and oracle.inq_n1(0.74) == -1
    Z = np.zeros(4, np.float32)
    assert oracle.Inq(4, 4, (), "largest_abs").quantize_weights(Z, np.ones(4, np.int32)) == (0, -3)


def test_inq_largest_abs_selection_and_state():
    """test_inq_affine.py:53-62: at an INQ iteration half of the learnable weights (largest |w|) become fixed;
    fixed weights are restored from the function's snapshot on later calls (inq_affine.cpp:95-102)."""
    rng = np.random.RandomState(1)
    W = (rng.randn(10, 10) * 0.1).astype(np.float32)
    I = np.zeros(W.shape, np.int32)
    inq = oracle.Inq(W.size, 4, (0, 2, 3), "largest_abs")
    W0 = W.copy()
    inq.quantize_weights(W, I)
    order = np.argsort(-np.abs(W0.ravel()), kind="stable")
    assert I.sum() == 50 and set(np.flatnonzero(I.ravel())) == set(order[:50])
    assert np.array_equal(W.ravel()[I.ravel() == 0], W0.ravel()[I.ravel() == 0])      # learnable ones untouched
    fixed_vals = W.copy()
    inq.commit(W, I)
    W += 0.01                                                                         # an "update" of every weight
    inq.quantize_weights(W, I)                                                        # counter 1: not an INQ step
    assert I.sum() == 50 and np.array_equal(W[I == 1], fixed_vals[I == 1])            # fixed weights restored
    inq.commit(W, I)
    inq.quantize_weights(W, I)                                                        # counter 2: fix half of the rest
    assert I.sum() == 75
    inq.commit(W, I)
    inq.quantize_weights(W, I)                                                        # counter 3 = last: fix all
    assert I.sum() == 100 and inq.counter == 3
    n_levels = np.unique(np.abs(W)).size
    assert n_levels <= 2 ** 2 + 1 + 4      # levels of up to three different ranges (max|w| changed between steps)


def test_inq_random_selection_is_seeded_bernoulli():
    W = np.linspace(-1, 1, 4000).astype(np.float32)
    runs = []
    for _ in range(2):
        inq = oracle.Inq(W.size, 4, (0, 5), "random", seed=42)
        Wc, I = W.copy(), np.zeros(W.shape, np.int32)
        inq.quantize_weights(Wc, I)
        runs.append(I.copy())
    assert np.array_equal(runs[0], runs[1]) and 1700 < runs[0].sum() < 2300
    with pytest.raises(oracle.OracleError):
        oracle.Inq(4, 4, (), "smallest")


def test_inq_affine_and_convolution_forward():
    rng = np.random.RandomState(2)
    x = rng.randn(6, 20).astype(np.float32)
    W = (rng.randn(20, 8) * 0.05).astype(np.float32)
    b = rng.randn(8).astype(np.float32)
    inq = oracle.Inq(W.size, 4, (0,), "largest_abs")
    Wq, I = W.copy(), np.zeros(W.shape, np.int32)
    y = inq.affine(x, Wq, I, b)
    ref_w, _, _ = _inq_quantize64(W, np.abs(W).max(), 4)
    assert max_rel_err(y, x.astype(np.float64) @ ref_w + b) < 3e-6 and inq.counter == 1
    xc = rng.randn(2, 3, 6, 6).astype(np.float32)
    Wc = (rng.randn(4, 3, 3, 3) * 0.05).astype(np.float32)
    inq = oracle.Inq(Wc.size, 4, (0,), "largest_abs")
    Wcq, Ic = Wc.copy(), np.zeros(Wc.shape, np.int32)
    yc = inq.convolution(xc, Wcq, Ic, None, (1, 1))
    ref_wc, _, _ = _inq_quantize64(Wc, np.abs(Wc).max(), 4)
    assert max_rel_err(yc, _torch_conv(xc, ref_wc.astype(np.float32), None, (1, 1), (1, 1), (1, 1), 1)) < 3e-6
