"""The drop-in path end to end on the GPU: ``F.*`` under the hip extension context -> nbla function registry ->
HipCachedArray storage -> C-ABI kernels, checked against the CPU oracle (the stand-in for nnabla's CPU context)."""
import numpy as np
import pytest

import nnabla_amd as nn
import nnabla_amd.functions as F
import oracle
from nnabla_amd import ext_hip
from nnabla_amd.ext_utils import get_extension_context
from util import bits_equal, first_mismatch, max_rel_err

pytestmark = pytest.mark.gpu
TOL, TIGHT = 1e-4, 5e-6


@pytest.fixture()
def ctx(dev):
    c = get_extension_context('hip', device_id='0')
    with nn.context_scope(c):
        yield c


def _var(a, dtype=None):
    v = nn.Variable(a.shape)
    if dtype is None:
        v.d = a
    else:
        v.set_data(a, dtype)
    return v


def test_extension_module_api(ctx):
    assert ext_hip.get_device_count() >= 1 and ext_hip.get_devices()[0] == '0'
    ext_hip.device_synchronize('0')
    ext_hip.synchronize(device_id='0')
    ext_hip.clear_memory_cache()


def test_fixed_point_and_pow2_quantize(ctx):
    rng = np.random.RandomState(313)
    x = (rng.randn(2, 3, 4) * 2).astype(np.float32)       # the reference tests' shape
    xv = _var(x)
    y = F.fixed_point_quantize(xv, True, 8, 2 ** -4)
    assert y.parent.name == 'FixedPointQuantize'
    y.forward()
    assert y.head_array_class == 'HipCachedArray'          # computed and left on the device
    assert bits_equal(y.d, oracle.fixed_point_quantize(x, True, 8, 2 ** -4))
    big = (rng.randn(64, 4099) * 3).astype(np.float32)
    for sign, n, delta in [(True, 8, 2 ** -4), (False, 5, 0.3), (True, 3, 0.1)]:
        y = F.fixed_point_quantize(_var(big), sign, n, delta)
        y.forward()
        assert bits_equal(y.d, oracle.fixed_point_quantize(big, sign, n, delta))
    w = (rng.randn(64, 32, 3, 3) * 0.05).astype(np.float32)
    for sign, wz, n, m in [(True, True, 4, 1), (False, False, 3, 0), (True, False, 8, 2)]:
        y = F.pow2_quantize(_var(w), sign, wz, n, m)
        y.forward()
        assert bits_equal(y.d, oracle.pow2_quantize(w, sign, wz, n, m))


def test_reforward_after_input_update_and_reshape(ctx):
    """The same graph re-run after the host rewrites the input (H2D sync again) and after a reshape (re-setup,
    function.cpp:107-123)."""
    rng = np.random.RandomState(1)
    xv = nn.Variable((5, 7))
    y = F.fixed_point_quantize(xv)
    for _ in range(2):
        x = (rng.randn(5, 7) * 2).astype(np.float32)
        xv.d = x
        y.forward()
        assert bits_equal(y.d, oracle.fixed_point_quantize(x))
    xv.reset_shape((3, 11), force=True)
    x = (rng.randn(3, 11) * 2).astype(np.float32)
    xv.d = x
    y.forward()
    assert y.shape == (3, 11) and bits_equal(y.d, oracle.fixed_point_quantize(x))


@pytest.mark.parametrize("xshape,qshape", [((4, 8, 16, 16), (1, 1, 1, 1)), ((4, 8, 16, 16), (1, 8, 1, 1)),
                                           ((16, 8, 3, 3), (16, 1, 1, 1))])
@pytest.mark.parametrize("x_min_max,ema", [(True, True), (True, False), (False, False)])
def test_min_max_quantize_updates_state_in_place(ctx, xshape, qshape, x_min_max, ema):
    rng = np.random.RandomState(313)
    qmn, qmx = np.full(qshape, -6, np.float32), np.full(qshape, 6, np.float32)
    lmn, lmx = np.zeros(qshape, np.float32), np.full(qshape, 255, np.float32)
    vmn, vmx = _var(qmn), _var(qmx)
    xv = nn.Variable(xshape)
    y = F.min_max_quantize(xv, vmn, vmx, _var(lmn), _var(lmx), 0.9, x_min_max, ema)
    for _ in range(3):                                     # running min/max evolve over minibatches
        x = (rng.randn(*xshape) * 2).astype(np.float32)
        xv.d = x
        y.forward()
        ref_y, qmn, qmx, _ = oracle.min_max_quantize(x, qmn, qmx, lmn, lmx, 0.9, x_min_max, ema, 0.01)
        assert bits_equal(y.d, ref_y), first_mismatch(y.d, ref_y)
        assert bits_equal(vmn.d, qmn) and bits_equal(vmx.d, qmx)


def test_binary_affines_write_their_parameters(ctx):
    rng = np.random.RandomState(5)
    x = rng.randn(6, 4, 20).astype(np.float32)             # base_axis = 2
    W = (rng.randn(20, 3, 5) * 0.1).astype(np.float32)
    b = rng.randn(3, 5).astype(np.float32)
    wb, alpha = nn.Variable(W.shape), nn.Variable((15,))
    y = F.binary_weight_affine(_var(x), _var(W), wb, alpha, _var(b), base_axis=2)
    y.forward()
    ref_y, ref_wb, ref_alpha = oracle.binary_weight_affine(x.reshape(24, 20), W.reshape(20, 15), b.ravel(), 1.0)
    assert y.shape == (6, 4, 3, 5)
    assert bits_equal(wb.d.reshape(20, 15), ref_wb)
    np.testing.assert_allclose(alpha.d, ref_alpha, rtol=2e-6)
    assert max_rel_err(y.d.reshape(24, 15), ref_y) <= TIGHT
    wb2 = nn.Variable(W.shape)
    y = F.binary_connect_affine(_var(x), _var(W), wb2, None, base_axis=2, quantize_zero_to=-1.0)
    y.forward()
    ref_y, ref_wb = oracle.binary_connect_affine(x.reshape(24, 20), W.reshape(20, 15), None, -1.0)
    assert bits_equal(wb2.d.reshape(20, 15), ref_wb) and max_rel_err(y.d.reshape(24, 15), ref_y) <= TIGHT


def test_binary_convolutions(ctx):
    rng = np.random.RandomState(7)
    x = rng.randn(4, 8, 16, 16).astype(np.float32)
    W = (rng.randn(16, 8, 3, 3) * 0.05).astype(np.float32)
    b = rng.randn(16).astype(np.float32)
    wb, alpha = nn.Variable(W.shape), nn.Variable((16,))
    y = F.binary_weight_convolution(_var(x), _var(W), wb, alpha, _var(b), pad=(1, 1), stride=(2, 1))
    y.forward()
    ref_y, ref_wb, ref_alpha = oracle.binary_weight_convolution(x, W, b, (1, 1), (2, 1), None, 1, 1.0)
    assert y.shape == ref_y.shape and bits_equal(wb.d, ref_wb)
    np.testing.assert_allclose(alpha.d, ref_alpha, rtol=2e-6)
    assert max_rel_err(y.d, ref_y) <= TIGHT
    wb2 = nn.Variable(W.shape)
    y = F.binary_connect_convolution(_var(x), _var(W), wb2, None, pad=(1, 1), group=1)
    y.forward()
    ref_y, ref_wb = oracle.binary_connect_convolution(x, W, None, (1, 1), None, None, 1, 1.0)
    assert bits_equal(wb2.d, ref_wb) and max_rel_err(y.d, ref_y) <= TIGHT


@pytest.mark.parametrize("algo", ["largest_abs", "random"])
def test_inq_affine_state_lives_in_the_function(ctx, algo):
    """The minibatch counter, the snapshot and the generator belong to the function object (inq_affine.hpp:86-92);
    float32 indicators written by the host are converted to int32 on first use, as in nnabla."""
    rng = np.random.RandomState(3)
    x = rng.randn(9, 40).astype(np.float32)
    W = (rng.randn(40, 24) * 0.05).astype(np.float32)
    its, seed = (0, 1, 3), 21
    inq = oracle.Inq(W.size, 4, its, algo, seed)
    Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
    wv, iv = _var(W), _var(np.zeros(W.shape, np.float32))
    y = F.inq_affine(_var(x), wv, iv, None, 1, 4, its, algo, seed)
    for it in range(5):
        ref_y = inq.affine(x, Wc, Ic, None)
        y.forward()
        assert np.array_equal(iv.d.astype(np.int32), Ic), "indicators differ at minibatch %d" % it
        assert bits_equal(wv.d, Wc)
        assert max_rel_err(y.d, ref_y) <= TIGHT
        upd = (rng.randn(*W.shape) * 0.01).astype(np.float32)
        Wc += upd
        wv.d = wv.d + upd
    y.forward()
    before, w_before = y.d.copy(), wv.d.copy()
    y.parent.recompute()                                    # product only: weights and counter stay as they are
    assert bits_equal(y.d, before) and bits_equal(wv.d, w_before)


def test_inq_convolution(ctx):
    rng = np.random.RandomState(4)
    x = rng.randn(2, 4, 9, 9).astype(np.float32)
    W = (rng.randn(6, 4, 3, 3) * 0.05).astype(np.float32)
    inq = oracle.Inq(W.size, 4, (0,), "largest_abs")
    Wc, Ic = W.copy(), np.zeros(W.shape, np.int32)
    ref_y = inq.convolution(x, Wc, Ic, None, (1, 1))
    wv, iv = _var(W), _var(np.zeros(W.shape, np.int32), np.int32)
    y = F.inq_convolution(_var(x), wv, iv, None, pad=(1, 1), num_bits=4, inq_iterations=(0,))
    y.forward()
    assert bits_equal(wv.d, Wc) and np.array_equal(iv.d, Ic) and max_rel_err(y.d, ref_y) <= TIGHT


def test_auto_forward_and_relu(ctx):
    x = (np.random.RandomState(2).randn(4, 9) * 2).astype(np.float32)
    with nn.auto_forward():
        y = F.relu(F.fixed_point_quantize(_var(x)))
        got = y.d
    ref = np.maximum(oracle.fixed_point_quantize(x), 0)
    assert np.array_equal(got, ref) and not np.signbit(got).any()


def test_device_memory_is_cached_and_released(ctx):
    ext_hip.clear_memory_cache()
    base = ext_hip.allocated_bytes('0')
    x = np.ones((1024, 1024), np.float32)
    y = F.fixed_point_quantize(_var(x))
    y.forward()
    _ = y.d
    held = ext_hip.allocated_bytes('0')
    assert held - base >= 2 * x.nbytes                      # input and output copies live on the device
    y2 = F.fixed_point_quantize(_var(x))
    y2.forward()
    del y, y2
    import gc
    gc.collect()
    ext_hip.clear_memory_cache()
    assert ext_hip.allocated_bytes('0') <= base + (1 << 20)


def _prove_chain_parity(gpu, ref, delta=2.0 ** -4, gemm_tol=5e-6, out_tol=TOL):
    """Proof that two runs of the quantized MLP (lists of (kind, [batch, width] output), entry 0 the common input)
    differ only by FixedPointQuantize tie flips.

    Rows of an MLP are independent, so a row is *clean* at a stage while no quantizer upstream has given the two runs
    different outputs in that row.  On clean rows the two runs feed every product bit-identical operands, so
      * what reaches the next quantizer differs by the summation-order error of one product only:
        |g - r| <= gemm_tol * max|r|;
      * where the quantizer outputs then differ, they differ by exactly one level, and the two pre-quantizer values
        lie on either side of (or on) the same rounding tie (k + 1/2) * delta -- the one thing an error that small can do
        to a step function;
      * the final outputs agree to out_tol of max|y|.
    Anything else (a product off by 1e-3, a quantizer off by a level away from a tie) fails an assertion.  Returns
    (fraction of rows clean at the end, flips per quantizer stage, worst clean-row output error)."""
    assert [k for k, _ in gpu] == [k for k, _ in ref] and gpu[0][0] == "input"
    batch = gpu[0][1].shape[0]
    clean = np.ones(batch, bool)
    flips = []
    for i in range(1, len(gpu)):
        kind, g_out = gpu[i]
        r_out = ref[i][1]
        g_in, r_in = gpu[i - 1][1], ref[i - 1][1]
        if kind == "fpq":
            scale = np.abs(r_in).max()
            d_in = np.abs(g_in[clean].astype(np.float64) - r_in[clean])
            assert d_in.max() <= gemm_tol * scale, \
                "stage %d: quantizer inputs of flip-free rows differ by %.3e of max|h|" % (i, d_in.max() / scale)
            mism = (g_out != r_out) & clean[:, None]
            rows, cols = np.nonzero(mism)
            if rows.size:
                go, ro = g_out[rows, cols].astype(np.float64), r_out[rows, cols].astype(np.float64)
                gi, ri = g_in[rows, cols].astype(np.float64), r_in[rows, cols].astype(np.float64)
                assert np.all(np.abs(go - ro) == delta), "stage %d: a mismatch of more than one level" % i
                assert np.all(np.sign(gi) * np.sign(ri) >= 0), "stage %d: mismatch across zero" % i
                tie = (np.floor(np.abs(gi) / delta) + 0.5) * delta      # the only tie within delta / 2 of |g_in|
                straddle = (np.abs(gi) - tie) * (np.abs(ri) - tie) <= 0
                assert np.all(straddle), "stage %d: %d mismatches that do not straddle a rounding tie" % (
                    i, int((~straddle).sum()))
                assert np.all(np.abs(np.abs(gi) - tie) <= gemm_tol * scale)
            flips.append(int(rows.size))
            clean &= ~mism.any(1)
        else:
            scale = np.abs(r_out).max()
            d = np.abs(g_out[clean].astype(np.float64) - r_out[clean])
            assert d.max() <= gemm_tol * scale, \
                "stage %d (%s): flip-free rows differ by %.3e of max|y|" % (i, kind, d.max() / scale)
    y_g, y_r = gpu[-1][1], ref[-1][1]
    worst = np.abs(y_g[clean].astype(np.float64) - y_r[clean]).max() / np.abs(y_r).max()
    assert worst <= out_tol, worst
    return clean.mean(), flips, worst


def test_config5_quantized_mlp_graph(ctx):
    """Benchmark configuration 5: batch 1024; FixedPointQuantize -> INQAffine 4096x4096 (num_bits 4, every weight fixed)
    -> 3 x [ReLU -> FixedPointQuantize -> BinaryWeightAffine 4096x4096]; x ~ N(0,1), W ~ N(0, 0.02^2).

    Per layer, with the oracle fed the same input the GPU layer saw (all rows): quantizer outputs, Wb and INQ weights
    are bit-exact, product outputs within 1e-4.  End to end against the oracle-only chain: the quantizers are step
    functions, so the ~1e-6 relative differences between two fp32 summation orders move a few activations across a
    rounding tie by one level (2^-4).  _prove_chain_parity asserts that this is the *only* difference: every
    mismatch is a one-level flip at a tie reached within the product's error, and every row without such a flip
    upstream agrees to 1e-4 (in fact 5e-6) at every stage and at the output.  The reference's own whole-graph metric
    (utils/cli/compare_with_cpu.py:46-52, std of the difference over the larger std) is printed beside it."""
    rng = np.random.default_rng(313)
    B, D = 1024, 4096
    x = rng.standard_normal((B, D), dtype=np.float32)
    Ws = [rng.standard_normal((D, D), dtype=np.float32) * np.float32(0.02) for _ in range(4)]
    # --- graph on the hip context
    xv = _var(x)
    w0, i0 = _var(Ws[0]), _var(np.zeros((D, D), np.float32))
    h = F.fixed_point_quantize(xv, True, 8, 2 ** -4)
    stages = [("fpq", h)]
    h = F.inq_affine(h, w0, i0, None, 1, 4, (0,), 'largest_abs')
    stages.append(("inq", h))
    wbs, alphas, wvs = [], [], []
    for l in range(1, 4):
        h = F.relu(h)
        stages.append(("relu", h))
        h = F.fixed_point_quantize(h, True, 8, 2 ** -4)
        stages.append(("fpq", h))
        wv, wb, al = _var(Ws[l]), nn.Variable((D, D)), nn.Variable((D,))
        wvs.append(wv), wbs.append(wb), alphas.append(al)
        h = F.binary_weight_affine(h, wv, wb, al)
        stages.append(("bwa", h))
    h.forward()
    gpu = [("input", x)] + [(kind, v.d) for kind, v in stages]
    # --- per-layer parity on identical inputs (all rows), and the oracle-only chain
    inq = oracle.Inq(D * D, 4, (0,), 'largest_abs')
    Wq, Iq = Ws[0].copy(), np.zeros((D, D), np.int32)
    cur_gpu_in, cur_ref = x, x
    ref = [("input", x)]
    layer = 0
    worst_gemm = 0.0
    for kind, out in gpu[1:]:
        if kind == "fpq":
            assert bits_equal(out, oracle.fixed_point_quantize(cur_gpu_in, True, 8, 2 ** -4))
            cur_ref = oracle.fixed_point_quantize(cur_ref, True, 8, 2 ** -4)
        elif kind == "relu":
            assert np.array_equal(out, np.maximum(cur_gpu_in, 0))
            cur_ref = np.maximum(cur_ref, 0)
        elif kind == "inq":
            same_chain = bits_equal(cur_ref, cur_gpu_in)
            ref_same_in = inq.affine(cur_gpu_in, Wq, Iq, None)     # quantizes Wq in place
            assert bits_equal(w0.d, Wq), first_mismatch(w0.d, Wq)
            assert np.array_equal(i0.d.astype(np.int32), Iq)
            worst_gemm = max(worst_gemm, max_rel_err(out, ref_same_in))
            cur_ref = ref_same_in if same_chain else oracle.affine(cur_ref, Wq)
        else:
            ref_same_in, ref_wb, ref_alpha = oracle.binary_weight_affine(cur_gpu_in, Ws[layer + 1], None, 1.0)
            assert bits_equal(wbs[layer].d, ref_wb)
            np.testing.assert_allclose(alphas[layer].d, ref_alpha, rtol=2e-6)
            worst_gemm = max(worst_gemm, max_rel_err(out, ref_same_in))
            cur_ref = oracle.affine(cur_ref, ref_wb * ref_alpha[None, :])
            layer += 1
        ref.append((kind, cur_ref))
        cur_gpu_in = out
    assert worst_gemm <= TOL, worst_gemm
    # --- end to end: the only differences are tie flips, and flip-free rows agree to 1e-4
    clean_frac, flips, worst_clean = _prove_chain_parity(gpu, ref)
    assert clean_frac >= 0.9, clean_frac
    y_gpu, y_cpu = gpu[-1][1], ref[-1][1]
    std_metric = np.std(y_gpu.astype(np.float64) - y_cpu) / max(np.std(y_gpu), np.std(y_cpu))
    print("config5: per-layer product max rel err %.2e (all rows, same inputs); end to end: %.1f%% of rows free of "
          "tie flips agree to %.2e of max|y|; tie flips per quantizer stage %s; reference's std metric over all rows "
          "%.2e, max-norm over all rows %.2e (diagnostics)" % (
              worst_gemm, 100 * clean_frac, worst_clean, flips, std_metric, max_rel_err(y_gpu, y_cpu)))
    # --- the proof has teeth: an error of 1e-3 in one layer's output (whole layer, or one element) is refused
    k = [i for i, (kind, _) in enumerate(gpu) if kind == "bwa"][1]
    scaled = list(gpu)
    scaled[k] = ("bwa", gpu[k][1] * np.float32(1.001))
    with pytest.raises(AssertionError):
        _prove_chain_parity(scaled, ref)
    poked = list(gpu)
    one = gpu[k][1].copy()
    one[17, 1234] += np.float32(1e-3) * np.abs(one).max()
    poked[k] = ("bwa", one)
    with pytest.raises(AssertionError):
        _prove_chain_parity(poked, ref)
    last = list(gpu)
    last[-1] = ("bwa", gpu[-1][1] * np.float32(1.001))
    with pytest.raises(AssertionError):
        _prove_chain_parity(last, ref)


# ------------------------------------------------------------------ backward
def test_quantizer_backward_through_the_registry(ctx):
    """F.* forward, Variable.backward(): the hip:float classes' backward_impl against the oracle, including the
    accumulation of leaf gradients and propagate_down."""
    rng = np.random.RandomState(5)
    x = rng.randn(6, 50).astype(np.float32) * 4
    gy = rng.randn(6, 50).astype(np.float32)
    if True:
        v = nn.Variable.from_numpy_array(x, need_grad=True)
        v.zero_grad()
        y = F.fixed_point_quantize(v, True, 4, 0.5, True)
        y.forward()
        y.backward(gy)
        ref = oracle.fixed_point_quantize_backward(gy, x, True, 4, 0.5, True)
        assert bits_equal(v.g, ref)
        y.backward(gy)                       # leaf gradients accumulate
        assert bits_equal(v.g, oracle.fixed_point_quantize_backward(gy, x, True, 4, 0.5, True, dx=ref))

        w = nn.Variable.from_numpy_array(x, need_grad=True)
        w.zero_grad()
        z = F.pow2_quantize(w, True, True, 4, 1, True)
        z.forward()
        z.backward(gy)
        # the leaf gradient was zero and is accumulated onto: 0 + (-0) = +0
        assert bits_equal(w.g, oracle.pow2_quantize_backward(gy, x, True, True, 4, 1, True, dx=np.zeros_like(x)))


def test_min_max_quantize_backward_through_the_registry(ctx):
    rng = np.random.RandomState(6)
    x = rng.randn(4, 3, 8, 8).astype(np.float32) * 3
    gy = rng.randn(4, 3, 8, 8).astype(np.float32)
    q = lambda v: np.full((1, 3, 1, 1), v, np.float32)
    if True:
        vx = nn.Variable.from_numpy_array(x, need_grad=True)
        vmin = nn.Variable.from_numpy_array(q(-2.0), need_grad=True)
        vmax = nn.Variable.from_numpy_array(q(2.0), need_grad=True)
        vlmin, vlmax = nn.Variable.from_numpy_array(q(0.0)), nn.Variable.from_numpy_array(q(255.0))
        for v in (vx, vmin, vmax):
            v.zero_grad()
        y = F.min_max_quantize(vx, vmin, vmax, vlmin, vlmax, 0.999, False, False, True, 0.01)
        y.forward()
        y.backward(gy)
        _, qmn, qmx, scale = oracle.min_max_quantize(x, q(-2.0), q(2.0), q(0.0), q(255.0), 0.999, False, False, 0.01)
        rdx, rmin, rmax = oracle.min_max_quantize_backward(gy, x, qmn, qmx, q(0.0), q(255.0), scale, True, False, False,
                                                           dx=np.zeros_like(x))
        assert bits_equal(vx.g, rdx)
        np.testing.assert_allclose(vmin.g, rmin, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(vmax.g, rmax, rtol=1e-5, atol=1e-5)


def test_quantized_mlp_backward(ctx):
    """Two quantized layers, forward and backward through the graph: gradients of the input and of both weight
    matrices against the oracle's chain (quantizer STEs bit-exact given the same upstream gradient; products at
    the fp32-faithful tolerance)."""
    rng = np.random.RandomState(17)
    B, D, H, O = 48, 96, 160, 40
    x = rng.randn(B, D).astype(np.float32)
    W1 = (rng.randn(D, H) * 0.05).astype(np.float32)
    W2 = (rng.randn(H, O) * 0.05).astype(np.float32)
    b2 = rng.randn(O).astype(np.float32)
    gy = rng.randn(B, O).astype(np.float32)

    vx = nn.Variable.from_numpy_array(x, need_grad=True)
    vW1 = nn.Variable.from_numpy_array(W1, need_grad=True)
    vW2 = nn.Variable.from_numpy_array(W2, need_grad=True)
    vb2 = nn.Variable.from_numpy_array(b2, need_grad=True)
    for v in (vx, vW1, vW2, vb2):
        v.zero_grad()
    q1 = F.fixed_point_quantize(vx, True, 8, 2.0 ** -4)
    a1 = F.binary_weight_affine(q1, vW1, nn.Variable(W1.shape), nn.Variable((H,)))
    h = F.relu(a1)
    q2 = F.fixed_point_quantize(h, True, 8, 2.0 ** -4)
    y = F.binary_connect_affine(q2, vW2, nn.Variable(W2.shape), vb2)
    y.forward()
    y.backward(gy)

    # oracle chain on the values the GPU produced (so that quantizer ties cannot diverge the two chains)
    oq1 = oracle.fixed_point_quantize(x, True, 8, 2.0 ** -4)
    assert bits_equal(q1.d, oq1)
    alpha1 = np.abs(W1).mean(0).astype(np.float32)
    ha, hq = h.d, q2.d
    g_q2, g_W2, g_b2 = oracle.binary_affine_backward(gy, hq, W2, None, 1.0)
    g_h = oracle.fixed_point_quantize_backward(g_q2, ha, True, 8, 2.0 ** -4, True)
    g_a1 = np.where(ha > 0, g_h, 0).astype(np.float32)
    g_q1, g_W1, _ = oracle.binary_affine_backward(g_a1, oq1, W1, alpha1, 1.0, want=(True, True, False))
    g_x = oracle.fixed_point_quantize_backward(g_q1, x, True, 8, 2.0 ** -4, True)
    assert max_rel_err(vW2.g, g_W2) <= TIGHT
    assert max_rel_err(vb2.g, g_b2) <= TIGHT
    assert max_rel_err(vW1.g, g_W1) <= TIGHT * 2
    assert max_rel_err(vx.g, g_x) <= TIGHT * 2
    # the clipped inputs receive exactly zero gradient
    clipped = (x > 7.9375) | (x < -7.9375)
    assert not vx.g[clipped].any()


def test_inq_affine_backward_through_the_registry(ctx):
    rng = np.random.RandomState(18)
    B, D, O = 20, 64, 96
    x = rng.randn(B, D).astype(np.float32)
    W = (rng.randn(D, O) * 0.05).astype(np.float32)
    gy = rng.randn(B, O).astype(np.float32)
    vx = nn.Variable.from_numpy_array(x, need_grad=True)
    vW = nn.Variable.from_numpy_array(W, need_grad=True)
    vI = nn.Variable(W.shape)
    vI.set_data(np.ones(W.shape), np.int32)
    vx.zero_grad()
    vW.zero_grad()
    y = F.inq_affine(vx, vW, vI, None, 1, 4, (), "largest_abs", -1)
    y.forward()
    y.backward(gy)
    Wq = vW.d                                   # quantized in place by the forward pass
    rdx, rdw, _ = oracle.affine_backward(gy, x, Wq, want=(True, True, False))
    assert max_rel_err(vx.g, rdx) <= TIGHT
    assert max_rel_err(vW.g, rdw) <= TIGHT


def test_convolution_backward_through_the_registry(ctx):
    """BinaryWeightConvolution -> ReLU -> BinaryConnectConvolution -> INQConvolution, backward through the graph."""
    rng = np.random.RandomState(19)
    x = rng.randn(3, 4, 10, 9).astype(np.float32)
    W1 = (rng.randn(8, 4, 3, 3) * 0.05).astype(np.float32)
    b1 = rng.randn(8).astype(np.float32)
    W2 = (rng.randn(6, 4, 3, 2) * 0.05).astype(np.float32)
    W3 = (rng.randn(5, 6, 2, 2) * 0.05).astype(np.float32)
    vx, vW1, vb1, vW2, vW3 = [nn.Variable.from_numpy_array(a, need_grad=True) for a in (x, W1, b1, W2, W3)]
    for v in (vx, vW1, vb1, vW2, vW3):
        v.zero_grad()
    vI = nn.Variable(W3.shape)
    vI.set_data(np.ones(W3.shape), np.int32)
    alpha1 = nn.Variable((8,))
    c1 = F.binary_weight_convolution(vx, vW1, nn.Variable(W1.shape), alpha1, vb1, pad=(1, 1), stride=(2, 1))
    h = F.relu(c1)
    c2 = F.binary_connect_convolution(h, vW2, nn.Variable(W2.shape), None, pad=(1, 0), group=2)
    y = F.inq_convolution(c2, vW3, vI, None, num_bits=4, inq_iterations=())
    y.forward()
    gy = rng.randn(*y.shape).astype(np.float32)
    y.backward(gy)

    hv, c2v, W3q = h.d, c2.d, vW3.d
    g_c2, g_W3, _ = oracle.convolution_backward(gy, c2v, W3q, want=(True, True, False))
    g_h, g_W2, _ = oracle.binary_convolution_backward(g_c2, hv, W2, None, (1, 0), None, None, 2, 1.0,
                                                      want=(True, True, False))
    g_c1 = np.where(hv > 0, g_h, 0).astype(np.float32)
    g_x, g_W1, g_b1 = oracle.binary_convolution_backward(g_c1, x, W1, alpha1.d, (1, 1), (2, 1), None, 1, 1.0)
    assert max_rel_err(vW3.g, g_W3) <= TIGHT
    assert max_rel_err(vW2.g, g_W2) <= TIGHT * 2
    assert max_rel_err(vW1.g, g_W1) <= TIGHT * 4
    assert max_rel_err(vb1.g, g_b1) <= TIGHT * 4
    assert max_rel_err(vx.g, g_x) <= TIGHT * 4


def test_quantize_dequantize_linear_and_prune_through_the_registry(ctx):
    rng = np.random.RandomState(23)
    x = (rng.randn(4, 6, 5, 5) * 3).astype(np.float32)
    scale = (np.abs(rng.randn(1, 6, 1, 1)) + 0.05).astype(np.float32)
    zp = (rng.randn(1, 6, 1, 1) * 4).astype(np.float32)
    vx = nn.Variable.from_numpy_array(x, need_grad=True)
    vx.zero_grad()
    vs, vz = _var(scale), _var(zp)
    p = F.prune(vx, rate=0.4)
    q = F.quantize_linear(p, vs, vz, 'HALF_TO_EVEN', True, np.int8)
    y = F.dequantize_linear(q, vs, vz)
    y.forward()
    rp = oracle.prune(x, 0.4)
    rq, rzp = oracle.quantize_linear(rp, scale, zp, 'HALF_TO_EVEN', True, 1)
    assert bits_equal(p.d, rp) and bits_equal(q.d, rq)
    assert bits_equal(vz.d, rzp)                                   # the zero point was rounded in place ...
    assert bits_equal(y.d, oracle.dequantize_linear(rq, scale, rzp))   # ... and the dequantizer sees the rounded one
    gy = rng.randn(*x.shape).astype(np.float32)
    y.backward(gy)
    g = oracle.linear_quantize_backward(oracle.linear_quantize_backward(gy, scale, True), scale, False)
    assert bits_equal(vx.g, g)                                     # Prune passes the gradient through
    with pytest.raises(ValueError):
        F.quantize_linear(vx, vs, vz, 'HALF_UP')
    with pytest.raises(ValueError):
        F.quantize_linear(vx, vs, _var(np.zeros((1, 5, 1, 1), np.float32)))
    with pytest.raises(ValueError):
        F.prune(vx, rate=1.5)
