"""The allocation-free MinMaxQuantize entry point (fixed per-device scratch inside the library) against the
workspace-taking entry point it is a variant of: bit-identical outputs and state, on consecutive calls that share
the scratch (the later ones smaller, so stale words of the earlier ones are in the array), and against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, first_mismatch, to_np

pytestmark = pytest.mark.gpu


def _dev(x, dev):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _both(dev, x, qshape, x_min_max, ema, decay=0.999, eps=0.01):
    """One call through each entry point on the same inputs; returns the two result tuples as numpy arrays."""
    qmn = np.full(qshape, -6.0, np.float32)
    qmx = np.full(qshape, 6.0, np.float32)
    lmn = np.full(qshape, 0.0, np.float32)
    lmx = np.full(qshape, 255.0, np.float32)
    xd = _dev(x, dev)
    # existing entry point (workspace from the caller)
    a_mn, a_mx = _dev(qmn, dev), _dev(qmx, dev)
    a_y, a_sc = kernels.min_max_quantize(xd, a_mn, a_mx, _dev(lmn, dev), _dev(lmx, dev), decay, x_min_max, ema, eps)
    # allocation-free entry point: every buffer, outputs included, exists before the call
    b_mn, b_mx = _dev(qmn, dev), _dev(qmx, dev)
    b_y = torch.full_like(xd, float("nan"))
    b_sc = torch.full_like(b_mn, float("nan"))
    l_mn, l_mx = _dev(lmn, dev), _dev(lmx, dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    kernels.min_max_quantize_static(xd, b_mn, b_mx, l_mn, l_mx, b_sc, b_y, decay, x_min_max, ema, eps)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before  # torch's allocator was not asked either
    ref = oracle.min_max_quantize(x, qmn, qmx, lmn, lmx, decay, x_min_max, ema, eps)
    return ((to_np(a_y), to_np(a_mn), to_np(a_mx), to_np(a_sc)),
            (to_np(b_y), to_np(b_mn), to_np(b_mx), to_np(b_sc)), ref)


def _check(dev, xshape, qshape, x_min_max, ema, seed):
    rng = np.random.RandomState(seed)
    x = (rng.randn(*xshape) * 3).astype(np.float32)
    a, b, ref = _both(dev, x, qshape, x_min_max, ema)
    for got_a, got_b, r, name in zip(a, b, ref, ("y", "qr_min", "qr_max", "scale")):
        assert bits_equal(got_b, got_a), "%s vs workspace entry: %s" % (name, first_mismatch(got_b, got_a))
        assert bits_equal(got_b, r), "%s vs oracle: %s" % (name, first_mismatch(got_b, r))


def test_static_scratch_two_calls_second_smaller(dev):
    """Per-tensor range with the EMA reduction: a large call, then a smaller one on the same scratch."""
    _check(dev, (8, 64, 56, 56), (1, 1, 1, 1), True, True, 313)
    _check(dev, (3, 5, 7, 9), (1, 1, 1, 1), True, True, 314)
    _check(dev, (1, 1, 1, 3), (1, 1, 1, 1), True, False, 315)


def test_static_scratch_per_channel_then_fewer_channels(dev):
    """Per-channel ranges (many partial rows in the scratch), then fewer channels, then no reduction at all."""
    _check(dev, (4, 512, 9, 8), (1, 512, 1, 1), True, True, 316)
    _check(dev, (4, 8, 16, 16), (1, 8, 1, 1), True, False, 317)
    _check(dev, (16, 8, 4, 4), (16, 1, 1, 1), True, True, 318)
    _check(dev, (6, 10), (1, 10), False, False, 319)
    _check(dev, (2, 3, 4), (2, 3, 4), True, True, 320)


def test_static_scratch_ranges_per_channel_and_column(dev):
    """Ranges of shape (1, C, 1, W): the workspace entry splits the reduction of every range over several blocks; with
    4096 ranges those partial results (2 MiB) do not fit the fixed scratch, and the allocation-free entry folds each
    range in one block instead.  Same bits; then a small case of the same kind."""
    _check(dev, (64, 64, 4, 64), (1, 64, 1, 64), True, True, 321)
    _check(dev, (3, 4, 5, 6), (1, 4, 1, 6), True, False, 322)


def test_static_scratch_rejects_what_does_not_fit(dev):
    """More quantization ranges than the fixed array holds: a clear error, nothing launched."""
    K = 8192 + 64
    x = torch.zeros((2, K), device=dev)
    q = torch.zeros((1, K), device=dev)
    need = kernels.lib().nbla_hip_min_max_quantize_workspace_bytes(kernels._shape(x.shape), 2, kernels._shape(q.shape))
    assert need > 256 * 1024
    y, sc = torch.empty_like(x), torch.empty_like(q)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.min_max_quantize_static(x, q.clone(), q.clone() + 1, q.clone(), q.clone() + 255, sc, y, 0.999, True,
                                        True)
    assert ei.value.code == kernels.ERR_MEMORY and "allocation-free" in str(ei.value)
    # the largest shape that does fit still works and matches
    _check(dev, (2, 8192), (1, 8192), True, True, 321)


def test_static_scratch_shape_error_as_the_workspace_entry(dev):
    x = torch.zeros((4, 6), device=dev)
    q = torch.zeros((1, 5), device=dev)
    with pytest.raises(kernels.KernelError) as ei:
        kernels.min_max_quantize_static(x, q, q.clone(), q.clone(), q.clone(), q.clone(), torch.empty_like(x))
    assert ei.value.code == kernels.ERR_VALUE
