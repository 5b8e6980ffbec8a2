"""INQAffine / INQConvolution on the GPU against the CPU oracle: quantized weights and indicators bit-exact over a
sequence of minibatches (restore, selection, quantization, snapshot), outputs within 1e-4 (expected ~1e-6)."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, first_mismatch, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TOL, TIGHT = 1e-4, 5e-6


def _dev(x, dev):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _step_for(counter, inq_iterations, algo):
    """The host-side mapping of inq_affine.cpp:104-113 from the minibatch counter to the C-ABI's step."""
    if counter in inq_iterations:
        if inq_iterations[-1] == counter:
            return kernels.INQ_FIX_ALL
        return kernels.INQ_LARGEST_ABS if algo == "largest_abs" else kernels.INQ_RANDOM
    return kernels.INQ_NO_SELECTION


def _cut_point_values(n):
    """Weights on and around the 1.5 * 2^k decision points and the pruning thresholds."""
    ks = np.arange(-12, 3)
    base = (1.5 * 2.0 ** ks).astype(np.float32)
    vals = [base, np.nextafter(base, np.float32(0)), np.nextafter(base, np.float32(9)), (2.0 ** ks).astype(np.float32),
            np.nextafter((2.0 ** ks).astype(np.float32), np.float32(0))]
    v = np.concatenate(vals)
    v = np.concatenate([v, -v, np.array([0.0, -0.0], np.float32)])
    return np.resize(v, n).astype(np.float32)


@pytest.mark.parametrize("num_bits", [2, 3, 4, 6])
@pytest.mark.parametrize("algo", ["largest_abs", "random"])
def test_inq_weight_sequence_matches_oracle(dev, num_bits, algo):
    rng = np.random.RandomState(313)
    shape = (70, 45)
    W = (rng.randn(*shape) * 0.05).astype(np.float32)
    W.ravel()[:200] = _cut_point_values(200) * 0.1
    its = (0, 2, 3, 5)
    seed = 11
    inq = oracle.Inq(W.size, num_bits, its, algo, seed)
    stream = oracle.Bernoulli(seed)
    Wc, Ic = W.copy(), np.zeros(shape, np.int32)
    Wd, Id = _dev(W, dev), torch.zeros(shape, dtype=torch.int32, device=dev)
    oldW, oldI = torch.zeros_like(Wd), torch.zeros_like(Id)
    for it in range(7):
        n1, n2 = inq.quantize_weights(Wc, Ic)
        inq.commit(Wc, Ic)
        step = _step_for(it, its, algo)
        n1n2 = kernels.inq_update_weights(Wd, Id, oldW, oldI, num_bits, step, draw=stream.draw)
        assert tuple(to_np(n1n2)) == (n1, n2)
        assert np.array_equal(to_np(Id), Ic), "indicators differ at minibatch %d" % it
        assert bits_equal(to_np(Wd), Wc), "minibatch %d: %s" % (it, first_mismatch(to_np(Wd), Wc))
        assert bits_equal(to_np(oldW), Wc) and np.array_equal(to_np(oldI), Ic)
        # the "optimizer" moves every weight; fixed ones must come back on the next forward
        upd = (rng.randn(*shape) * 0.01).astype(np.float32)
        Wc += upd
        Wd += _dev(upd, dev)
    assert Ic.min() == 1


def test_inq_largest_abs_tie_free_half_selection(dev):
    """Exactly the num_learnable // 2 largest |w| become fixed, including the single-element quirk of the loop."""
    for size in (1, 2, 3, 101, 4096):
        rng = np.random.RandomState(size)
        W = (rng.permutation(size).astype(np.float32) + 1) * np.where(rng.rand(size) < 0.5, -1, 1) * 0.001
        W = W.astype(np.float32)
        inq = oracle.Inq(size, 4, (0, 9), "largest_abs")
        Wc, Ic = W.copy(), np.zeros(size, np.int32)
        inq.quantize_weights(Wc, Ic)
        Wd, Id = _dev(W, dev), torch.zeros(size, dtype=torch.int32, device=dev)
        kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), 4, kernels.INQ_LARGEST_ABS)
        assert np.array_equal(to_np(Id), Ic) and bits_equal(to_np(Wd), Wc)
        assert Ic.sum() == max(size // 2, 1)


@pytest.mark.parametrize("size,offset", [(7, 0), (1000, 0), (4099, 1), (70001, 0), (262147, 3), (1 << 21, 0)])
@pytest.mark.parametrize("distinct", [1, 3, 40])
def test_inq_largest_abs_with_many_equal_magnitudes(dev, size, offset, distinct):
    """Weights drawn from a handful of magnitudes, part of them already fixed: std::sort leaves the order of equal
    magnitudes to the library (inq_affine.cpp:121-123), so the comparison with the oracle is per magnitude -- the
    number of newly fixed weights of every magnitude -- plus what the selection itself promises: num_learnable // 2
    are fixed, none of them smaller than a weight left learnable, and among the weights of the magnitude where the
    selection stops the lowest indices are taken.  `offset` moves the arrays off 16-byte alignment."""
    rng = np.random.RandomState(size + distinct)
    mags = (0.001 * (1 + np.arange(distinct))).astype(np.float32)
    W = (mags[rng.randint(0, distinct, size)] * np.where(rng.rand(size) < 0.5, -1, 1)).astype(np.float32)
    I0 = (rng.rand(size) < 0.3).astype(np.int32)
    inq = oracle.Inq(size, 4, (0, 9), "largest_abs")
    Wc, Ic = W.copy(), I0.copy()
    inq.quantize_weights(Wc, Ic)
    Wd = torch.zeros(size + offset, dtype=torch.float32, device=dev)[offset:]
    Id = torch.zeros(size + offset, dtype=torch.int32, device=dev)[offset:]
    Wd.copy_(_dev(W, dev)), Id.copy_(_dev(I0, dev))
    kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), 4, kernels.INQ_LARGEST_ABS)
    Ig = to_np(Id)
    learnable = I0 == 0
    T = int(learnable.sum()) // 2
    new_g, new_c = (Ig == 1) & learnable, (Ic == 1) & learnable
    assert np.array_equal(Ig[~learnable], I0[~learnable])
    assert new_g.sum() == new_c.sum() == max(T, int(new_c.sum()))
    a = np.abs(W)
    for m in mags:
        assert (new_g & (a == m)).sum() == (new_c & (a == m)).sum(), "magnitude %g" % m
    if new_g.any() and (learnable & ~new_g).any():
        stop = a[new_g].min()
        assert stop >= a[learnable & ~new_g].max()
        ties = np.flatnonzero(learnable & (a == stop))
        taken = int(new_g[ties].sum())
        assert new_g[ties[:taken]].all() and not new_g[ties[taken:]].any()
    # the weights fixed by both are quantized alike
    both = (Ig == 1) & (Ic == 1)
    assert bits_equal(to_np(Wd)[both], Wc[both])


def test_inq_largest_abs_with_one_learnable_weight(dev):
    """num_learnable // 2 == 0: the loop of inq_affine.cpp:133-141 still looks at the first index of the sorted
    order and fixes it if it is learnable, i.e. only when the one learnable weight has the largest magnitude."""
    for size, where, largest in ((1, 0, True), (5, 3, True), (5, 3, False), (3000, 2999, True), (3000, 17, False)):
        W = np.linspace(0.01, 0.02, size).astype(np.float32)
        W[where] = 0.5 if largest else 0.001
        I0 = np.ones(size, np.int32)
        I0[where] = 0
        inq = oracle.Inq(size, 4, (0, 9), "largest_abs")
        Wc, Ic = W.copy(), I0.copy()
        inq.quantize_weights(Wc, Ic)
        Wd, Id = _dev(W, dev), _dev(I0, dev)
        kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), 4, kernels.INQ_LARGEST_ABS)
        assert Ic[where] == int(largest)
        assert np.array_equal(to_np(Id), Ic), (size, where, largest)
        assert bits_equal(to_np(Wd), Wc)
    # nothing learnable at all
    W, I0 = np.full(9, 0.3, np.float32), np.ones(9, np.int32)
    Wd, Id = _dev(W, dev), _dev(I0, dev)
    kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), 4, kernels.INQ_LARGEST_ABS)
    assert to_np(Id).min() == 1


@pytest.mark.parametrize("size,offset", [(5, 0), (4099, 1), (300001, 0)])
def test_inq_random_selection_draw_order(dev, size, offset):
    """Learnable weight number r in index order takes draw r of the stream (inq_affine.cpp:143-149), for any
    alignment and for sizes above one chunk of the ranking kernels."""
    rng = np.random.RandomState(size)
    W = (rng.randn(size) * 0.05).astype(np.float32)
    I0 = (rng.rand(size) < 0.4).astype(np.int32)
    inq = oracle.Inq(size, 4, (0, 9), "random", 5)
    stream = oracle.Bernoulli(5)
    Wc, Ic = W.copy(), I0.copy()
    inq.quantize_weights(Wc, Ic)
    Wd = torch.zeros(size + offset, dtype=torch.float32, device=dev)[offset:]
    Id = torch.zeros(size + offset, dtype=torch.int32, device=dev)[offset:]
    Wd.copy_(_dev(W, dev)), Id.copy_(_dev(I0, dev))
    kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), 4, kernels.INQ_RANDOM,
                               draw=stream.draw)
    assert np.array_equal(to_np(Id), Ic) and bits_equal(to_np(Wd), Wc)


@pytest.mark.parametrize("num_bits,top", [(4, 1.9), (6, 1.4)])
def test_inq_every_weight_of_the_level_range(dev, num_bits, top):
    """Every fp32 value from below the pruning threshold up to max|w| (whole binades, both signs), all fixed:
    the quantized weights follow the host libm's log2f cut for cut (inq_affine.cpp:153-190)."""
    lo_exp, hi_exp = (-6, 0) if num_bits == 4 else (-18, 0)
    for e in range(lo_exp, hi_exp + 1):
        u = np.arange(1 << 23, dtype=np.uint32) | np.uint32((e + 127) << 23)
        w = u.view(np.float32).copy()
        w[1::2] *= -1
        w[0] = np.float32(top)  # the same max|w| (hence n1, n2) for every binade
        w = w[np.abs(w) <= np.float32(top)]
        inq = oracle.Inq(w.size, num_bits, (0,), "largest_abs")
        Wc, Ic = w.copy(), np.zeros(w.size, np.int32)
        n1, n2 = inq.quantize_weights(Wc, Ic)
        Wd, Id = _dev(w, dev), torch.zeros(w.size, dtype=torch.int32, device=dev)
        n1n2 = kernels.inq_update_weights(Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), num_bits,
                                          kernels.INQ_FIX_ALL)
        assert tuple(to_np(n1n2)) == (n1, n2)
        assert bits_equal(to_np(Wd), Wc), "binade 2^%d: %s" % (e, first_mismatch(to_np(Wd), Wc))
        assert int(to_np(Id).min()) == 1


@pytest.mark.parametrize("M,K,N", [(2, 3, 4), (33, 100, 130), (64, 256, 192), (300, 520, 257)])
def test_inq_affine_all_fixed_and_partially_fixed(dev, M, K, N):
    rng = np.random.RandomState(5)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    for its, nsteps in (((0,), 1), ((0, 5), 2)):        # all fixed at once / half fixed then a plain minibatch
        inq = oracle.Inq(W.size, 4, its, "largest_abs")
        Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
        Wd, Id = _dev(W, dev), torch.zeros(W.shape, dtype=torch.int32, device=dev)
        oldW, oldI = torch.zeros_like(Wd), torch.zeros_like(Id)
        for it in range(nsteps):
            ref_y = inq.affine(x, Wc, Ic, b)
            y = kernels.inq_affine(_dev(x, dev), Wd, Id, oldW, oldI, _dev(b, dev), 4,
                                   _step_for(it, its, "largest_abs"))
            assert bits_equal(to_np(Wd), Wc) and np.array_equal(to_np(Id), Ic)
            y64 = x.astype(np.float64) @ Wc.astype(np.float64) + b
            assert max_rel_err(to_np(y), ref_y) <= TOL
            assert max_rel_err(to_np(y), y64) <= TIGHT
        # recompute: the product alone on the weights left by the forward
        y2 = kernels.inq_affine(_dev(x, dev), Wd, Id, oldW, oldI, _dev(b, dev), 4, kernels.INQ_PRODUCT_ONLY)
        assert bits_equal(to_np(y2), to_np(y)) and bits_equal(to_np(Wd), Wc)


@pytest.mark.parametrize("num_bits", [3, 4, 5])
@pytest.mark.parametrize("K,N", [(256, 32), (512, 96), (768, 288)])
def test_inq_affine_one_digit_weights_with_columns_of_different_reach(dev, K, N, num_bits):
    """The weight operand of the product takes its one-digit form when every weight is zero or a power of two and no
    column spans more than six binades: with every weight fixed at num_bits <= 4 (seven levels at most) it does, with
    num_bits 5 the levels of a column can span more, and with weights still being learnt there are values that are no
    powers of two: both take the three-digit form.  Columns of very different magnitude (some entirely below the top
    level's reach, some pruned to zero) are part of the data.  The forward's product (column statistics gathered by
    the quantizing pass) must give the bits of the product-only call (statistics from a pass of its own) and agree
    with the oracle."""
    rng = np.random.RandomState(K + N + num_bits)
    M = 40
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    W[:, ::5] *= np.float32(2.0 ** -3)                  # columns whose largest level lies below the global one
    W[:, 3::7] *= np.float32(2.0 ** -9)                 # columns pruned to zero, or out of one digit's reach
    W[::3, 1] = 0.0
    b = rng.randn(N).astype(np.float32)
    for its, nsteps in (((0,), 1), ((0, 5), 2)):        # all fixed at once / half fixed then a plain minibatch
        inq = oracle.Inq(W.size, num_bits, its, "largest_abs")
        Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
        Wd, Id = _dev(W, dev), torch.zeros(W.shape, dtype=torch.int32, device=dev)
        oldW, oldI = torch.zeros_like(Wd), torch.zeros_like(Id)
        for it in range(nsteps):
            ref_y = inq.affine(x, Wc, Ic, b)
            y = kernels.inq_affine(_dev(x, dev), Wd, Id, oldW, oldI, _dev(b, dev), num_bits,
                                   _step_for(it, its, "largest_abs"))
            assert bits_equal(to_np(Wd), Wc) and np.array_equal(to_np(Id), Ic)
            y64 = x.astype(np.float64) @ Wc.astype(np.float64) + b
            assert max_rel_err(to_np(y), ref_y) <= TOL
            assert max_rel_err(to_np(y), y64) <= TIGHT
            y2 = kernels.inq_affine(_dev(x, dev), Wd, Id, oldW, oldI, _dev(b, dev), num_bits,
                                    kernels.INQ_PRODUCT_ONLY)
            assert bits_equal(to_np(y2), to_np(y)) and bits_equal(to_np(Wd), Wc)


@pytest.mark.parametrize("M,K,N", [(8, 256, 192), (5, 100, 130)])   # with / without the column-statistics pass
def test_inq_affine_steady_state_writes_only_what_changes(dev, M, K, N):
    """Once the snapshot holds every weight as fixed, the quantizing pass leaves alone what the restoring pass of the
    same call has just copied from the snapshot and quantization does not change.  That must stay invisible:
    forwards after an optimizer step that moved every weight, after the snapshot's values were replaced by numbers
    that are no powers of two (they have to be quantized and written back), and after indicators were cleared again
    behind the function's back (the snapshot's indicators have to follow) all leave W, I and the snapshot as the
    oracle's."""
    rng = np.random.RandomState(21)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.02).astype(np.float32)
    inq = oracle.Inq(W.size, 4, (0,), "largest_abs")
    Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
    Wd, Id = _dev(W, dev), torch.zeros(W.shape, dtype=torch.int32, device=dev)
    oldW, oldI = torch.zeros_like(Wd), torch.zeros_like(Id)

    def forward(step):
        ref_y = inq.affine(x, Wc, Ic, None)
        y = kernels.inq_affine(_dev(x, dev), Wd, Id, oldW, oldI, None, 4, step)
        assert bits_equal(to_np(Wd), Wc), first_mismatch(to_np(Wd), Wc)
        assert np.array_equal(to_np(Id), Ic)
        assert bits_equal(to_np(oldW), Wc) and np.array_equal(to_np(oldI), Ic)
        assert max_rel_err(to_np(y), ref_y) <= TOL

    forward(kernels.INQ_FIX_ALL)
    assert Ic.min() == 1
    for _ in range(2):                                    # the optimizer moves every weight; all of them come back
        upd = (rng.randn(K, N) * 0.01).astype(np.float32)
        Wc += upd
        Wd += _dev(upd, dev)
        forward(kernels.INQ_NO_SELECTION)
    # the snapshot's values replaced in places: restored as they are, then quantized and written everywhere
    snap = Wc.copy()
    snap[::3, ::5] = (rng.randn(*snap[::3, ::5].shape) * 0.01).astype(np.float32)
    inq.commit(snap, Ic)
    oldW.copy_(_dev(snap, dev))
    forward(kernels.INQ_NO_SELECTION)
    # indicators cleared behind the function's back: those weights are learnable again, the snapshot must say so
    Ic[1::4, 2::3] = 0
    Id.copy_(_dev(Ic, dev))
    upd = (rng.randn(K, N) * 0.01).astype(np.float32)
    Wc += upd
    Wd += _dev(upd, dev)
    forward(kernels.INQ_NO_SELECTION)
    assert Ic.min() == 0
    forward(kernels.INQ_NO_SELECTION)                     # and a forward with a snapshot that is no longer all fixed


def test_inq_convolution_matches_oracle(dev):
    rng = np.random.RandomState(9)
    for xs, ws, pad, stride, group in [((2, 4, 9, 9), (6, 4, 3, 3), (1, 1), (1, 1), 1),
                                       ((3, 6, 8, 7), (4, 3, 3, 2), (1, 0), (2, 1), 2)]:
        x = rng.randn(*xs).astype(np.float32)
        W = (rng.randn(*ws) * 0.05).astype(np.float32)
        b = rng.randn(ws[0]).astype(np.float32)
        its = (0, 1)
        inq = oracle.Inq(W.size, 4, its, "largest_abs")
        Wc, Ic = W.copy(), np.zeros(ws, np.int32)
        Wd, Id = _dev(W, dev), torch.zeros(ws, dtype=torch.int32, device=dev)
        oldW, oldI = torch.zeros_like(Wd), torch.zeros_like(Id)
        for it in range(2):
            ref_y = inq.convolution(x, Wc, Ic, b, pad, stride, None, group)
            y = kernels.inq_convolution(_dev(x, dev), Wd, Id, oldW, oldI, _dev(b, dev), pad, stride, None, group, 4,
                                        _step_for(it, its, "largest_abs"))
            assert bits_equal(to_np(Wd), Wc) and np.array_equal(to_np(Id), Ic)
            assert max_rel_err(to_np(y), ref_y) <= TIGHT


def test_convolution_with_fixed_weights_takes_the_one_digit_form(dev):
    """Weights INQ has fixed are powers of two within seven binades: as a row-scaled digit operand each output
    channel is a one-digit row (its values whole units of the top digit), and a tile of the product whose 128
    channels are all of that kind multiplies three digit pairs instead of six.  Nothing is dropped either way, so the
    channels give the same bits when a general channel in their tile forces the six-pair form; and the result is
    the float64 convolution of x as rounded to 24 bits per window."""
    rng = np.random.RandomState(5)
    xs, ws = (3, 32, 12, 12), (160, 32, 3, 3)          # two tiles of output channels, the second partly empty
    x = rng.randn(*xs).astype(np.float32)
    e = rng.randint(-8, -2, size=ws)
    W = (np.where(rng.rand(*ws) < 0.2, 0.0, 2.0 ** e) * rng.choice([-1.0, 1.0], size=ws)).astype(np.float32)
    I = torch.ones(ws, dtype=torch.int32, device=dev)

    def run(Wh):
        Wd = _dev(Wh, dev)
        return to_np(kernels.inq_convolution(_dev(x, dev), Wd, I, Wd.clone(), I.clone(), None, (1, 1), (1, 1), None, 1,
                                             4, kernels.INQ_PRODUCT_ONLY))
    y1 = run(W)
    assert max_rel_err(y1, oracle.convolution(x, W, None, (1, 1), (1, 1), None, 1)) <= TIGHT
    W6 = W.copy()
    W6[::128] = (rng.randn(2, *ws[1:]) * 0.05).astype(np.float32)   # one general channel in each tile
    y6 = run(W6)
    same = np.ones(ws[0], bool)
    same[::128] = False
    assert bits_equal(y1[:, same], y6[:, same])
    assert max_rel_err(y6, oracle.convolution(x, W6, None, (1, 1), (1, 1), None, 1)) <= TIGHT


@pytest.mark.parametrize("xs,ws,pad,stride,group", [
    ((2, 8, 9, 9), (6, 8, 3, 3), (1, 1), (1, 1), 1),
    ((3, 6, 10, 7), (8, 3, 3, 2), (0, 1), (2, 1), 2),
])
def test_convolution_with_non_finite_values(dev, xs, ws, pad, stride, group):
    """A window of x or an output channel of W holding NaN / Inf: the outputs they reach are the reference's, one by
    one (convolution.cpp:185-193), the others those of the clean operands bit for bit; through the product-only step
    that Convolution runs, and through INQConvolution's forward with every weight still being learnt."""
    rng = np.random.RandomState(9)
    x = rng.randn(*xs).astype(np.float32)
    W = (rng.randn(*ws) * 0.1).astype(np.float32)
    b = rng.randn(ws[0]).astype(np.float32)

    def run(xh, Wh, step):
        Wd = _dev(Wh, dev)
        I = torch.zeros(ws, dtype=torch.int32, device=dev)
        return to_np(kernels.inq_convolution(_dev(xh, dev), Wd, I, Wd.clone(), I.clone(), _dev(b, dev), pad, stride,
                                             None, group, 4, step))
    clean = run(x, W, kernels.INQ_PRODUCT_ONLY)
    x[1, 2, 4, 5] = np.inf
    x[1, 1, 4, 6] = np.inf
    x[0, 0, 0, 0] = np.nan
    x[1, 0, 8, 1] = -np.inf
    W[4, 1, 2, 0] = np.inf
    W[1, 0, 0, 1] = np.nan
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.convolution(x, W, b, pad, stride, None, group)
    y = run(x, W, kernels.INQ_PRODUCT_ONLY)
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert np.array_equal(np.isposinf(y), np.isposinf(ref)) and np.array_equal(np.isneginf(y), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert fin.any() and np.isnan(ref).any() and np.isinf(ref).any()
    assert bits_equal(y[fin], clean[fin])


def test_convolution_with_fixed_weights_at_the_resnet_stage_shape(dev):
    """Benchmark configuration 4's shape with power-of-two weights (98 tiles of the digit product, the contraction
    split over blocks, every tile in the one-digit form for its weights) against torch's float64 convolution."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(32, 256, 14, 14, generator=g)
    e = torch.randint(-8, -2, (256, 256, 3, 3), generator=g).float()
    W = torch.pow(2.0, e) * (torch.randint(0, 2, e.shape, generator=g).float() * 2 - 1)
    W[torch.rand(W.shape, generator=g) < 0.2] = 0.0
    b = torch.randn(256, generator=g)
    Wd, I = W.to(dev), torch.ones(W.shape, dtype=torch.int32, device=dev)
    y = kernels.inq_convolution(x.to(dev), Wd, I, Wd.clone(), I.clone(), b.to(dev), (1, 1), (1, 1), None, 1, 4,
                                kernels.INQ_PRODUCT_ONLY)
    ref = torch.nn.functional.conv2d(x.double().to(dev), W.double().to(dev), b.double().to(dev), padding=1)
    assert max_rel_err(to_np(y), ref.cpu().numpy()) <= TIGHT


def test_inq_config5_layer(dev):
    """The INQAffine layer of benchmark configuration 5: x [1024,4096], W [4096,4096] ~ N(0, 0.02^2), num_bits 4, every
    weight fixed.  Weights bit-exact against the oracle; the output against float64 on sampled entries and against
    the oracle's fp32 GEMM on the first 64 rows."""
    rng = np.random.default_rng(313)
    x = rng.standard_normal((1024, 4096), dtype=np.float32)
    W = rng.standard_normal((4096, 4096), dtype=np.float32) * np.float32(0.02)
    inq = oracle.Inq(W.size, 4, (0,), "largest_abs")
    Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
    ref_y = inq.affine(x[:64], Wc, Ic, None)
    Wd, Id = _dev(W, dev), torch.zeros(W.shape, dtype=torch.int32, device=dev)
    y = to_np(kernels.inq_affine(_dev(x, dev), Wd, Id, torch.zeros_like(Wd), torch.zeros_like(Id), None, 4,
                                 kernels.INQ_FIX_ALL))
    assert bits_equal(to_np(Wd), Wc), first_mismatch(to_np(Wd), Wc)
    assert np.array_equal(to_np(Id), Ic) and Ic.min() == 1
    assert max_rel_err(y[:64], ref_y) <= TOL
    rows, cols = rng.choice(1024, 32, replace=False), rng.choice(4096, 64, replace=False)
    ref = x[rows].astype(np.float64) @ Wc[:, cols].astype(np.float64)
    assert np.abs(y[np.ix_(rows, cols)] - ref).max() / np.abs(ref).max() <= TIGHT


def test_inq_affine_replays_in_a_hip_graph(dev):
    """INQAffine forward between selection steps (weights partly fixed, partly learnt) and once every weight is fixed,
    captured once each and replayed after the learnable weights and the input changed: the replay's output, weights
    and snapshot are those of the eager call (its passes clear and fill counters on the device and never
    synchronise)."""
    rng = np.random.RandomState(23)
    M, K, N = 96, 256, 384
    x = torch.empty(M, K, device=dev)
    for fix_all in (False, True):
        Wh = (rng.randn(K, N) * 0.05).astype(np.float32)
        W, I = _dev(Wh, dev), torch.zeros((K, N), dtype=torch.int32, device=dev)
        oW, oI = torch.zeros_like(W), torch.zeros_like(I)
        x.copy_(_dev(rng.randn(M, K).astype(np.float32), dev))
        # one selection step outside the capture: half of the weights (or all of them) become fixed
        kernels.inq_affine(x, W, I, oW, oI, None, 4, kernels.INQ_FIX_ALL if fix_all else kernels.INQ_LARGEST_ABS)
        kernels.inq_affine(x, W, I, oW, oI, None, 4, kernels.INQ_NO_SELECTION)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = kernels.inq_affine(x, W, I, oW, oI, None, 4, kernels.INQ_NO_SELECTION)
        for i in range(3):
            x.copy_(_dev((rng.randn(M, K) * (i + 1)).astype(np.float32), dev))
            # a training step moved the weights (the fixed ones are put back by the forward)
            W.add_(_dev((rng.randn(K, N) * 0.01).astype(np.float32), dev))
            before = [t.clone() for t in (W, I, oW, oI)]
            graph.replay()
            torch.cuda.synchronize()
            got = [to_np(t).copy() for t in (y, W, I, oW, oI)]
            for t, b in zip((W, I, oW, oI), before):
                t.copy_(b)
            ye = kernels.inq_affine(x, W, I, oW, oI, None, 4, kernels.INQ_NO_SELECTION)
            torch.cuda.synchronize()
            for g, e, name in zip(got, (ye, W, I, oW, oI), ("y", "W", "I", "old W", "old I")):
                assert bits_equal(g, to_np(e)), "fix_all %s replay %d: %s differs" % (fix_all, i, name)
            ref = to_np(x).astype(np.float64) @ to_np(W).astype(np.float64)
            assert np.abs(got[0] - ref).max() / np.abs(ref).max() <= TIGHT
