"""A seeded sweep over random convolution geometries (one to three spatial dimensions, strides, dilations, paddings,
groups, channel counts on both sides of what the LDS-slab product takes): the binary convolutions' forward against
the CPU oracle and their backward (input, weight and bias gradients) against the oracle's, at the fp32-faithful
tolerance.  The hand-picked cases of the other convolution tests name the corner each one is for; this one looks for
the corners nobody named."""
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


def _geometries(count, seed):
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        nd = int(rng.choice([1, 2, 2, 2, 3]))
        group = int(rng.choice([1, 1, 1, 2, 3]))
        cg = int(rng.choice([1, 3, 8, 24, 31, 32, 40, 48, 64, 96]))
        og = int(rng.choice([1, 5, 24, 32, 33, 70]))
        limit = {1: 60, 2: 14, 3: 7}[nd]
        in_sp = tuple(int(v) for v in rng.randint(1, limit + 1, size=nd))
        kernel = tuple(int(v) for v in rng.randint(1, 4, size=nd))
        dil = tuple(int(v) for v in rng.randint(1, 3, size=nd))
        stride = tuple(int(v) for v in rng.choice([1, 1, 2, 3], size=nd))
        pad = tuple(int(v) for v in rng.randint(0, 3, size=nd))
        if any(in_sp[i] + 2 * pad[i] < dil[i] * (kernel[i] - 1) + 1 for i in range(nd)):
            continue
        n = int(rng.choice([1, 2, 5]))
        work = n * group * cg * og * int(np.prod(in_sp)) * int(np.prod(kernel))
        if work > 6e7:   # keeps the CPU oracle to a second or two per case
            continue
        out.append(((n, group * cg) + in_sp, (group * og, cg) + kernel, pad, stride, dil, group))
    return out


GEOMETRIES = _geometries(48, 2718)


def test_the_sweep_reaches_both_forms():
    """Some geometries of the sweep take the product on input positions held in LDS, some the gathering one."""
    taken = [kernels.binary_convolution_slab_plan(xs[0], xs[1], xs[2:], ws[0], ws[2:], pad, stride, dil, group)
             is not None for xs, ws, pad, stride, dil, group in GEOMETRIES]
    assert 8 <= sum(taken) <= len(taken) - 8


@pytest.mark.parametrize("case", range(len(GEOMETRIES)))
def test_forward_and_backward(dev, case):
    xs, ws, pad, stride, dil, group = GEOMETRIES[case]
    print("geometry", xs, ws, pad, stride, dil, group, flush=True)
    rng = np.random.RandomState(1000 + case)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)
    ref_y, ref_Wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, pad, stride, dil, group, 1.0)
    d = lambda a: _dev(a, dev)
    y, Wb, alpha = kernels.binary_weight_convolution(d(x), d(W), d(b), pad, stride, dil, group)
    assert tuple(y.shape) == ref_y.shape
    assert bits_equal(to_np(Wb), ref_Wb)
    np.testing.assert_allclose(to_np(alpha), ref_alpha, rtol=2e-6)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT
    yc, Wbc = kernels.binary_connect_convolution(d(x), d(W), None, pad, stride, dil, group)
    ref_yc, _ = oracle.binary_connect_convolution(x, W, None, pad, stride, dil, group, 1.0)
    assert bits_equal(to_np(Wbc), ref_Wb)
    assert max_rel_err(to_np(yc), ref_yc) <= TIGHT

    dy = rng.randn(*ref_y.shape).astype(np.float32)
    rdx, rdw, rdb = oracle.binary_convolution_backward(dy, x, W, ref_alpha, pad, stride, dil, group, 1.0)
    gdx, gdw, gdb = kernels.binary_convolution_backward(d(dy), d(x), d(W), None, d(ref_alpha), pad, stride, dil, group,
                                                        1.0)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT


@pytest.mark.parametrize("case", range(0, len(GEOMETRIES), 2))
def test_real_weights_forward_and_backward(dev, case):
    """The digit x digit product of Convolution / INQConvolution (product only: the weights are left alone) and its
    backward on every other geometry of the sweep."""
    xs, ws, pad, stride, dil, group = GEOMETRIES[case]
    print("geometry", xs, ws, pad, stride, dil, group, flush=True)
    rng = np.random.RandomState(2000 + case)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.05).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)
    d = lambda a: _dev(a, dev)
    ref_y = oracle.convolution(x, W, b, pad, stride, dil, group)
    Wd = d(W)
    Id = torch.zeros(ws, dtype=torch.int32, device=dev)
    y = kernels.inq_convolution(d(x), Wd, Id, Wd.clone(), Id.clone(), d(b), pad, stride, dil, group, 4,
                                kernels.INQ_PRODUCT_ONLY)
    assert bits_equal(to_np(Wd), W)
    assert max_rel_err(to_np(y), ref_y) <= TIGHT
    dy = rng.randn(*ref_y.shape).astype(np.float32)
    rdx, rdw, rdb = oracle.convolution_backward(dy, x, W, pad, stride, dil, group)
    gdx, gdw, gdb = kernels.convolution_backward(d(dy), d(x), d(W), pad, stride, dil, group)
    for got, ref in ((gdx, rdx), (gdw, rdw), (gdb, rdb)):
        assert max_rel_err(to_np(got), ref) <= TIGHT
