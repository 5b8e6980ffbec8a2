"""A seeded sweep over random (M, K, N) of the binary affine functions, aligned and not: every form the forward's
dispatcher knows (one pass on the vector ALUs, one pass on bf16 matrix instructions, one walk with the signs through
LDS, two walks with packed bits) meets odd row counts, contractions that are no multiple of 4 / 16 / 32 and output
widths that end inside a vector, a fragment or a column group.  Forward against the CPU oracle (Wb bit for bit,
alpha at 2e-6, y at the fp32-faithful tolerance), backward against the oracle's gradients."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TIGHT = 5e-6


def _dev(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _shapes(count, seed):
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        M = int(rng.choice([1, 2, 7, 8, 9, 16, 31, 64, 65, 100, 128, 200, 256, 257, 400, 513]))
        K = int(rng.choice([1, 3, 4, 15, 16, 31, 32, 33, 64, 100, 250, 256, 1000, 1024, 2049]))
        N = int(rng.choice([1, 2, 4, 5, 31, 32, 33, 127, 128, 129, 255, 256, 260, 512, 1000, 2052]))
        if M * K * N > 3e8:
            continue
        out.append((M, K, N))
    return out


SHAPES = _shapes(60, 1618)


@pytest.mark.parametrize("case", range(len(SHAPES)))
def test_forward_and_backward(dev, case):
    M, K, N = SHAPES[case]
    print("shape", M, K, N, flush=True)
    rng = np.random.RandomState(3000 + case)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    d = lambda a: _dev(a, dev)
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_affine(x, W, b, 1.0)
    y, Wb, alpha = kernels.binary_weight_affine(d(x), d(W), d(b))
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT
    ref_yc, _ = oracle.binary_connect_affine(x, W, None, 1.0)
    yc, Wbc = kernels.binary_connect_affine(d(x), d(W))
    assert bits_equal(to_np(Wbc), ref_Wb)
    assert max_rel_err(to_np(yc), ref_yc) <= TIGHT

    dy = rng.randn(M, N).astype(np.float32)
    rdx, rdw, rdb = oracle.binary_affine_backward(dy, x, W, ref_alpha, 1.0)
    gdx, gdw, gdb = kernels.binary_affine_backward(d(dy), d(x), d(W), None, d(ref_alpha), 1.0)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT
