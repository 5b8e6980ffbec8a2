"""Element-wise quantizers on tensors of more than 2^31 elements (8.6 GB per tensor): indices and byte offsets past
what 32 bits hold, and an end that falls inside a vector and a block.  The input repeats one million-element period,
so the output must repeat the output of that period -- itself bit-checked against the CPU oracle -- and the
comparison stays on the device."""
import numpy as np
import pytest
import torch

import oracle
from nnabla_amd import kernels
from util import bits_equal, to_np

pytestmark = pytest.mark.gpu

@pytest.fixture(autouse=True)
def _release_device_memory():
    yield
    torch.cuda.empty_cache()   # the 8.6 GB tensors go back to the device, not into the caching allocator's pool


PERIOD = 1 << 20
N = (1 << 31) + 5 * PERIOD + 13   # not a multiple of 4: the tail past the last 16-byte vector


def _periodic(dev, seed, scale):
    base = (np.random.RandomState(seed).randn(PERIOD) * scale).astype(np.float32)
    base[::97] = 0.0
    base[5::101] = -0.0
    b = torch.from_numpy(base).to(dev)
    reps = N // PERIOD + 1
    x = b.repeat(reps)[:N].contiguous()
    return base, x


def _repeats(y, first):
    """y (length N) equals `first` (length PERIOD) repeated, bit for bit; compared in int32 on the device."""
    yi, fi = y.view(torch.int32), first.view(torch.int32)
    whole = (N // PERIOD) * PERIOD
    ok = bool((yi[:whole].view(-1, PERIOD) == fi).all())
    return ok and bool((yi[whole:] == fi[:N - whole]).all())


def test_fixed_point_and_pow2_quantize_past_2_31_elements(dev):
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * (1 << 30):
        pytest.skip("needs 40 GB of free device memory")
    base, x = _periodic(dev, 11, 2.0)
    y = kernels.fixed_point_quantize(x, True, 8, 2.0 ** -4)
    first = y[:PERIOD].clone()
    assert bits_equal(to_np(first), oracle.fixed_point_quantize(base, True, 8, 2.0 ** -4))
    assert _repeats(y, first)
    # backward on the same tensors: dy = y, fine-grained mask
    dx = kernels.fixed_point_quantize_backward(y, x, True, 8, 2.0 ** -4, True)
    ref = oracle.fixed_point_quantize_backward(to_np(first), base, True, 8, 2.0 ** -4, True)
    assert bits_equal(to_np(dx[:PERIOD]), ref)
    assert _repeats(dx, dx[:PERIOD].clone())
    del dx
    kernels.pow2_quantize(x, True, True, 4, 1, out=y)
    first = y[:PERIOD].clone()
    assert bits_equal(to_np(first), oracle.pow2_quantize(base, True, True, 4, 1))
    assert _repeats(y, first)


def test_min_max_quantize_past_2_31_elements(dev):
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * (1 << 30):
        pytest.skip("needs 40 GB of free device memory")
    base, x = _periodic(dev, 12, 3.0)
    q = lambda v: torch.full((1,), v, dtype=torch.float32, device=dev)
    qmn, qmx = q(-6.0), q(6.0)
    y, scale = kernels.min_max_quantize(x, qmn, qmx, q(0.0), q(255.0), 0.999, True, True)
    one = lambda v: np.full((1,), v, np.float32)
    ry, rmn, rmx, rscale = oracle.min_max_quantize(base, one(-6.0), one(6.0), one(0.0), one(255.0), 0.999, True, True,
                                                   0.01)
    # the extrema of the whole tensor are those of one period (first of equal zeros: inside the first period)
    assert bits_equal(to_np(qmn), rmn) and bits_equal(to_np(qmx), rmx) and bits_equal(to_np(scale), rscale)
    first = y[:PERIOD].clone()
    assert bits_equal(to_np(first), ry)
    assert _repeats(y, first)


def test_binary_weight_affine_output_past_2_31_elements(dev):
    """y of 70,000 x 32,768 (2.29e9 elements, 9.2 GB): output offsets beyond 32 bits in the product's stores.  Rows
    from both ends and the middle against float64."""
    free, _ = torch.cuda.mem_get_info()
    if free < 30 * (1 << 30):
        pytest.skip("needs 30 GB of free device memory")
    M, K, N = 70000, 64, 32768
    rng = np.random.RandomState(13)
    x = rng.randn(M, K).astype(np.float32)
    W = (rng.randn(K, N) * 0.05).astype(np.float32)
    b = rng.randn(N).astype(np.float32)
    y, Wb, alpha = kernels.binary_weight_affine(torch.from_numpy(x).to(dev), torch.from_numpy(W).to(dev),
                                                torch.from_numpy(b).to(dev))
    assert y.numel() > (1 << 31)
    ref_Wb = np.where(W < 0, np.float32(-1), np.float32(1))
    assert bits_equal(to_np(Wb), ref_Wb)
    Wd = ref_Wb.astype(np.float64) * np.abs(W.astype(np.float64)).mean(0)
    rows = [0, 1, 31, 32, 34999, 65535, 65536, 65537, 69998, 69999]
    got = to_np(y[rows])
    ref = x[rows].astype(np.float64) @ Wd + b
    assert np.abs(got - ref).max() / np.abs(ref).max() <= 5e-6
    # nothing but finite values anywhere (a store gone astray would leave the allocator's old bytes or fault)
    assert bool(torch.isfinite(y).all())


@pytest.mark.parametrize("M", [4, 48, 200, 600])
def test_binary_weight_affine_weights_past_2_31_elements(dev, M):
    """W of 36,000 x 65,536 (2.36e9 weights, 9.4 GB, and as much again for Wb) through each form of the forward: one
    pass on the vector ALUs, one pass on the matrix cores, one walk, two walks.  Checked on the device: Wb against
    the sign of W everywhere, alpha and y against float64 on the first and the last columns."""
    free, _ = torch.cuda.mem_get_info()
    if free < 50 * (1 << 30):
        pytest.skip("needs 50 GB of free device memory")
    K, N = 36000, 65536
    g = torch.Generator(device=dev).manual_seed(100 + M)
    W = torch.randn(K, N, generator=g, device=dev) * 0.05
    x = torch.randn(M, K, generator=g, device=dev)
    assert W.numel() > (1 << 31)
    y, Wb, alpha = kernels.binary_weight_affine(x, W)
    assert bool((Wb == torch.where(W < 0, -1.0, 1.0)).all())
    for cols in (slice(0, 384), slice(N - 384, N)):
        a64 = W[:, cols].double().abs().mean(0)
        assert float(((alpha[cols].double() - a64).abs() / a64).max()) <= 2e-6
        ref = x.double() @ (Wb[:, cols].double() * a64)
        err = float((y[:, cols].double() - ref).abs().max() / ref.abs().max())
        assert err <= 5e-6, err
    assert bool(torch.isfinite(y).all())


def test_binary_affine_backward_weights_past_2_31_elements(dev):
    """The same weight matrix through the backward pass: dW (2.36e9 outputs of the digit x digit product, a plain
    x^T dy under the straight-through estimator) and dx = (dy * alpha) Wb^T, against float64 on blocks from the
    corners of each result."""
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * (1 << 30):
        pytest.skip("needs 60 GB of free device memory")
    M, K, N = 320, 36000, 65536
    g = torch.Generator(device=dev).manual_seed(7)
    W = torch.randn(K, N, generator=g, device=dev) * 0.05
    x = torch.randn(M, K, generator=g, device=dev)
    dy = torch.randn(M, N, generator=g, device=dev)
    alpha = W.abs().mean(0)
    dx, dW, db = kernels.binary_affine_backward(dy, x, W, None, alpha, 1.0)
    assert dW.numel() > (1 << 31)
    for rows in (slice(0, 256), slice(K - 256, K)):
        for cols in (slice(0, 256), slice(N - 256, N)):
            ref = x[:, rows].double().t() @ dy[:, cols].double()
            err = float((dW[rows, cols].double() - ref).abs().max() / ref.abs().max())
            assert err <= 5e-6, err
    for rows in (slice(0, 512), slice(K - 512, K)):
        Wb = torch.where(W[rows] < 0, -1.0, 1.0).double()
        ref = (dy.double() * alpha.double()) @ Wb.t()
        err = float((dx[:, rows].double() - ref).abs().max() / ref.abs().max())
        assert err <= 5e-6, err
    ref = dy.double().sum(0)
    assert float((db.double() - ref).abs().max() / ref.abs().max()) <= 5e-6
    assert bool(torch.isfinite(dW).all())


def test_quantize_and_dequantize_linear_past_2_31_elements(dev):
    """A [rows, 2^20] tensor of more than 2^31 elements with a per-column scale (the broadcast index arithmetic of
    the two functions) and with one scale for the whole tensor (QuantizeLinear's own fast path)."""
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * (1 << 30):
        pytest.skip("needs 40 GB of free device memory")
    rows = (1 << 11) + 3
    rng = np.random.RandomState(14)
    base = (rng.randn(1, PERIOD) * 30).astype(np.float32)
    x = torch.from_numpy(base).to(dev).repeat(rows, 1).contiguous()
    assert x.numel() > (1 << 31)
    col_scale = (0.1 + rng.rand(1, PERIOD)).astype(np.float32)
    col_zp = rng.randint(-3, 4, size=(1, PERIOD)).astype(np.float32)
    for scale, zp in ((col_scale, col_zp), (np.full((1, 1), 0.3, np.float32), np.full((1, 1), 2.0, np.float32))):
        y = kernels.quantize_linear(x, torch.from_numpy(scale).to(dev), torch.from_numpy(zp.copy()).to(dev),
                                    "HALF_TO_EVEN", False, kernels.DTYPE_BYTE)
        ref, _ = oracle.quantize_linear(base, scale, zp, "HALF_TO_EVEN", False, kernels.DTYPE_BYTE)
        assert bits_equal(to_np(y[0:1]), ref)
        assert bool((y.view(torch.int32) == y[0:1].view(torch.int32)).all())
        z = kernels.dequantize_linear(y, torch.from_numpy(scale).to(dev), torch.from_numpy(zp).to(dev))
        assert bits_equal(to_np(z[rows - 1:rows]), oracle.dequantize_linear(ref, scale, zp))
        assert bool((z.view(torch.int32) == z[0:1].view(torch.int32)).all())
        del y, z
