"""GPU parity of the affine backward passes (BinaryWeightAffine, BinaryConnectAffine, Affine/INQAffine) against the
CPU oracle at the north-star tolerance and against float64 at the fp32-faithful one."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TOL, TIGHT = 1e-4, 5e-6


def _dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _data(M, K, N, seed):
    rng = np.random.RandomState(seed)
    return (rng.randn(M, K).astype(np.float32), (rng.randn(K, N) * 0.02).astype(np.float32),
            rng.randn(M, N).astype(np.float32))


SHAPES = [(1, 32, 64), (5, 17, 9), (33, 100, 130), (64, 256, 256), (300, 520, 257), (40, 70, 4096)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("with_alpha", [True, False])
def test_binary_affine_backward(dev, M, K, N, with_alpha):
    x, W, dy = _data(M, K, N, 31)
    alpha = np.abs(W).mean(0).astype(np.float32) if with_alpha else None
    rdx, rdw, rdb = oracle.binary_affine_backward(dy, x, W, alpha, 1.0)
    d = lambda a: None if a is None else _dev(a, dev)
    gdx, gdw, gdb = kernels.binary_affine_backward(d(dy), d(x), d(W), None, d(alpha), 1.0)
    sgn = np.where(W >= 0, 1.0, -1.0) * (alpha.astype(np.float64) if with_alpha else 1.0)
    dx64 = dy.astype(np.float64) @ sgn.T
    dw64 = x.astype(np.float64).T @ dy.astype(np.float64)
    db64 = dy.astype(np.float64).sum(0)
    for got, ref, ref64 in ((gdx, rdx, dx64), (gdw, rdw, dw64), (gdb, rdb, db64)):
        assert max_rel_err(to_np(got), ref) <= TOL
        assert max_rel_err(to_np(got), ref64) <= TIGHT
        assert max_rel_err(ref, ref64) <= TIGHT


def test_binary_affine_backward_accumulates_and_skips(dev):
    M, K, N = 37, 96, 200
    x, W, dy = _data(M, K, N, 32)
    alpha = np.abs(W).mean(0).astype(np.float32)
    rng = np.random.RandomState(3)
    odx, odw, odb = (rng.randn(M, K).astype(np.float32), rng.randn(K, N).astype(np.float32),
                     rng.randn(N).astype(np.float32))
    rdx, rdw, rdb = oracle.binary_affine_backward(dy, x, W, alpha, 1.0, dx=odx, dW=odw, db=odb)
    d = lambda a: _dev(a, dev)
    gdx, gdw, gdb = kernels.binary_affine_backward(d(dy), d(x), d(W), None, d(alpha), 1.0, dx=d(odx), dW=d(odw),
                                                   db=d(odb))
    assert max_rel_err(to_np(gdx), rdx) <= TIGHT
    assert max_rel_err(to_np(gdw), rdw) <= TIGHT
    assert max_rel_err(to_np(gdb), rdb) <= TIGHT
    only = kernels.binary_affine_backward(d(dy), d(x), d(W), None, d(alpha), 1.0, want=(False, True, False))
    assert only[0] is None and only[2] is None
    assert max_rel_err(to_np(only[1]), x.astype(np.float64).T @ dy.astype(np.float64)) <= TIGHT


@pytest.mark.parametrize("M,K,N", [(2048, 96, 130), (3000, 200, 64), (1500, 40, 520)])
def test_backward_small_outputs_long_batch(dev, M, K, N):
    """Few output tiles and a long contraction over the samples: the weight-gradient product spreads the contraction
    over the CUs (partial results summed in a fixed order), here onto gradients that are already there; so does the
    input gradient of a real-weight layer when N is the long index."""
    x, W, dy = _data(M, K, N, 35)
    rng = np.random.RandomState(5)
    odw = rng.randn(K, N).astype(np.float32)
    d = lambda a: _dev(a, dev)
    _, gdw, _ = kernels.binary_affine_backward(d(dy), d(x), d(W), None, None, 1.0, dW=d(odw), want=(False, True, False))
    dw64 = odw.astype(np.float64) + x.astype(np.float64).T @ dy.astype(np.float64)
    assert max_rel_err(to_np(gdw), dw64) <= TIGHT
    again = kernels.binary_affine_backward(d(dy), d(x), d(W), None, None, 1.0, dW=d(odw), want=(False, True, False))[1]
    assert bits_equal(to_np(again), to_np(gdw))                      # deterministic
    # real-weight dx with the roles exchanged: [N', K'] weights, contraction over the long index
    x2, W2, dy2 = _data(K, N, M, 36)                                 # dy2 [K, M], W2 [N, M]
    gdx = kernels.affine_backward(d(dy2), d(x2), d(W2), want=(True, False, False))[0]
    assert max_rel_err(to_np(gdx), dy2.astype(np.float64) @ W2.astype(np.float64).T) <= TIGHT


@pytest.mark.parametrize("q0", [0.0, 0.5, -1.0])
def test_binary_affine_backward_with_zero_weights(dev, q0):
    """Sign(0) = quantize_zero_to: values other than +-1 cannot be packed to one bit and take the general product."""
    M, K, N = 20, 64, 72
    x, W, dy = _data(M, K, N, 33)
    W.ravel()[::5] = 0.0
    alpha = np.abs(W).mean(0).astype(np.float32)
    Wb = oracle.sign(W, q0)
    rdx, rdw, _ = oracle.binary_affine_backward(dy, x, W, alpha, q0)
    d = lambda a: _dev(a, dev)
    gdx, gdw, _ = kernels.binary_affine_backward(d(dy), d(x), d(W), d(Wb), d(alpha), q0)
    assert max_rel_err(to_np(gdx), rdx) <= TIGHT * 4
    assert max_rel_err(to_np(gdw), rdw) <= TIGHT * 4


@pytest.mark.parametrize("zeros", [False, True])
@pytest.mark.parametrize("M,K,N", [(20, 64, 72), (300, 200, 130)])
def test_binary_affine_backward_zero_to_decided_on_the_device(dev, M, K, N, zeros):
    """quantize_zero_to = 0 onto a gradient that is already there: with exact-zero weights the fp32 product over the
    signs must be the one that adds to dx, without them the bit-weight product -- exactly one of the two, chosen on
    the device (the call never synchronises)."""
    x, W, dy = _data(M, K, N, 37)
    if zeros:
        W.ravel()[::5] = 0.0
    alpha = np.abs(W).mean(0).astype(np.float32)
    Wb = oracle.sign(W, 0.0)
    odx = np.random.RandomState(8).randn(M, K).astype(np.float32)
    d = lambda a: _dev(a, dev)
    gdx = kernels.binary_affine_backward(d(dy), d(x), d(W), d(Wb), d(alpha), 0.0, dx=d(odx),
                                         want=(True, False, False))[0]
    dx64 = odx.astype(np.float64) + (dy.astype(np.float64) * alpha) @ Wb.astype(np.float64).T
    assert max_rel_err(to_np(gdx), dx64) <= TIGHT * 4


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_affine_backward_real_weights(dev, M, K, N):
    """The product inside INQAffine: weights that are zero or signed powers of two, and arbitrary ones."""
    x, W, dy = _data(M, K, N, 34)
    for weights in (W, np.sign(W) * np.exp2(np.round(np.log2(np.abs(W) + 1e-9))).astype(np.float32)):
        weights = weights.astype(np.float32)
        rdx, rdw, rdb = oracle.affine_backward(dy, x, weights)
        d = lambda a: _dev(a, dev)
        gdx, gdw, gdb = kernels.affine_backward(d(dy), d(x), d(weights))
        dx64 = dy.astype(np.float64) @ weights.astype(np.float64).T
        assert max_rel_err(to_np(gdx), dx64) <= TIGHT and max_rel_err(to_np(gdx), rdx) <= TOL
        assert max_rel_err(to_np(gdw), x.astype(np.float64).T @ dy.astype(np.float64)) <= TIGHT
        assert max_rel_err(to_np(gdb), dy.astype(np.float64).sum(0)) <= TIGHT


def test_backward_full_size_sample(dev):
    """BinaryWeightAffine backward at K=4096, N=11008 with M=512: sampled rows / columns against float64."""
    M, K, N = 512, 4096, 11008
    rng = np.random.default_rng(9)
    x = rng.standard_normal((M, K), dtype=np.float32)
    W = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    dy = rng.standard_normal((M, N), dtype=np.float32)
    alpha = np.abs(W).mean(0).astype(np.float32)
    d = lambda a: _dev(a, dev)
    gdx, gdw, gdb = kernels.binary_affine_backward(d(dy), d(x), d(W), None, d(alpha), 1.0)
    rows, cols = rng.choice(M, 16, replace=False), rng.choice(K, 64, replace=False)
    ws = np.where(W[cols] >= 0, 1.0, -1.0) * alpha.astype(np.float64)
    ref = dy[rows].astype(np.float64) @ ws.T
    assert np.abs(to_np(gdx)[np.ix_(rows, cols)] - ref).max() / np.abs(ref).max() <= TIGHT
    ks, ns = rng.choice(K, 32, replace=False), rng.choice(N, 64, replace=False)
    ref = x[:, ks].astype(np.float64).T @ dy[:, ns].astype(np.float64)
    assert np.abs(to_np(gdw)[np.ix_(ks, ns)] - ref).max() / np.abs(ref).max() <= TIGHT
    assert max_rel_err(to_np(gdb), dy.astype(np.float64).sum(0)) <= TIGHT
