"""Quantization-aware training on the GPU: the range-recorder kernel against the CPU oracle (bit-exact), the recorder
functions through the registry, and the converted graphs end to end (recording graph == float graph; simulated-
quantization graph against the same chain computed with the oracle's functions)."""
import numpy as np
import pytest
import torch

import nnabla_amd as nn
import nnabla_amd.experimental.graph_converters as GC
import nnabla_amd.functions as F
import nnabla_amd.parametric_functions as PF
import oracle
from nnabla_amd import kernels as K
from nnabla_amd.ext_utils import get_extension_context
from nnabla_amd.utils import qnn
from nnabla_amd.utils.qnn import FunctionsRankRecorder, QATConfig, QATScheduler, QNNState
from util import bits_equal, first_mismatch, max_rel_err, to_np

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture()
def ctx(dev):
    nn.clear_parameters()
    with nn.context_scope(get_extension_context('hip', device_id='0')):
        yield
    nn.clear_parameters()


def _var(a):
    v = nn.Variable(a.shape)
    v.d = a
    return v


def _f32_bits(a):
    return np.asarray(a, np.float32).reshape(-1).view(np.uint32)


# ----------------------------------------------------------------------------------------------- kernel vs oracle
@pytest.mark.parametrize("kind", oracle.RECORDERS)
@pytest.mark.parametrize("shape", [(1,), (3,), (7, 9), (4, 16, 16), (1000, 1031), (2, 3, 1024, 1024)])
def test_recorder_kernel_bit_exact(dev, kind, shape):
    """Three consecutive batches: statistics and the copied output against the oracle, bit for bit."""
    rng = np.random.default_rng(1000 * oracle.RECORDERS.index(kind) + len(shape) + sum(shape))
    two = kind in ("MinMaxMinMaxRecorder", "MinMaxMvaRecorder")
    m_ref, M_ref = np.float32(0.0), np.float32(0.0)
    m = torch.zeros(1, device=dev) if two else None
    M = torch.zeros(1, device=dev)
    for it in range(3):
        x = (rng.standard_normal(shape) * (it + 1) + 0.25 * it).astype(np.float32)
        xt = torch.from_numpy(x).to(dev)
        y = K.range_recorder(xt, m, M, kind, decay=0.99)
        assert bits_equal(to_np(y), x), first_mismatch(to_np(y), x)
        m_ref, M_ref = oracle.range_recorder(x, m_ref if two else None, M_ref, kind, 0.99)
        assert _f32_bits(to_np(M))[0] == _f32_bits(M_ref)[0], (it, to_np(M), M_ref)
        if two:
            assert _f32_bits(to_np(m))[0] == _f32_bits(m_ref)[0], (it, to_np(m), m_ref)


@pytest.mark.parametrize("kind", ["MinMaxMvaRecorder", "AbsMaxRecorder"])
@pytest.mark.parametrize("x_off,y_off", [(1, 0), (0, 2), (3, 3), (1, None)])
def test_recorder_on_views_that_are_not_16_byte_aligned(dev, kind, x_off, y_off):
    """x or y starting at an odd multiple of four bytes (y_off None: in place): the same statistics and copy, through
    32-bit accesses spread over all the blocks."""
    rng = np.random.default_rng(5)
    n = 300007
    x = rng.standard_normal(n).astype(np.float32)
    x[1234] = -0.0
    xb = torch.zeros(n + 8, device=dev)
    xb[x_off:x_off + n] = torch.from_numpy(x).to(dev)
    xv = xb[x_off:x_off + n]
    yb = torch.full((n + 8,), 7.0, device=dev)
    yv = xv if y_off is None else yb[y_off:y_off + n]
    two = kind == "MinMaxMvaRecorder"
    m = torch.zeros(1, device=dev) if two else None
    M = torch.zeros(1, device=dev)
    y = K.range_recorder(xv, m, M, kind, decay=0.99, y=yv)
    m_ref, M_ref = oracle.range_recorder(x, np.float32(0.0) if two else None, np.float32(0.0), kind, 0.99)
    assert bits_equal(to_np(y), x)
    assert _f32_bits(to_np(M))[0] == _f32_bits(M_ref)[0]
    if two:
        assert _f32_bits(to_np(m))[0] == _f32_bits(m_ref)[0]
    if y_off is not None:
        assert (to_np(yb[:y_off]) == 7.0).all() and (to_np(yb[y_off + n:]) == 7.0).all()


def test_recorder_kernel_edge_cases(dev):
    """Signed zeros, NaNs, values beyond the +-1e8 the reductions start from, unaligned views, in-place, training off."""
    cases = [np.array([-0.0, 0.0, -0.0], np.float32), np.array([0.0, -0.0], np.float32),
             np.array([np.nan, 1.0, -2.0, np.nan], np.float32), np.full(5, np.nan, np.float32),
             np.array([3e8, -3e8], np.float32), np.array([-3e8, -2e8], np.float32),
             np.array([np.inf, -np.inf, 1.0], np.float32), np.zeros(1031, np.float32)]
    for x in cases:
        for kind in oracle.RECORDERS:
            two = kind in ("MinMaxMinMaxRecorder", "MinMaxMvaRecorder")
            for start in (0.0, -1.5, 2.5):
                m = torch.full((1,), start, device=dev) if two else None
                M = torch.full((1,), start, device=dev)
                K.range_recorder(torch.from_numpy(x).to(dev), m, M, kind, decay=0.9)
                m_ref, M_ref = oracle.range_recorder(x, start if two else None, start, kind, 0.9)
                assert bits_equal(to_np(M), [M_ref]), (x, kind, start, to_np(M), M_ref)
                if two:
                    assert bits_equal(to_np(m), [m_ref]), (x, kind, start, to_np(m), m_ref)
    rng = np.random.default_rng(3)
    base = torch.from_numpy(rng.standard_normal(4099).astype(np.float32)).to(dev)
    for off, n in [(1, 4096), (3, 1001), (2, 5)]:          # not 16-byte aligned
        view = base[off:off + n]
        M = torch.zeros(1, device=dev)
        y = torch.empty(n + 1, device=dev)[1:]
        K.range_recorder(view, None, M, "AbsMaxRecorder", y=y)
        assert bits_equal(to_np(y), to_np(view))
        assert to_np(M)[0] == np.abs(to_np(view)).max()
    x = base.clone()
    M = torch.zeros(1, device=dev)
    K.range_recorder(x, None, M, "MaxMaxRecorder", y=x)    # in place: no copy, statistics only
    assert bits_equal(to_np(x), to_np(base)) and to_np(M)[0] == to_np(base).max()
    M = torch.full((1,), 7.0, device=dev)
    y = K.range_recorder(base, None, M, "MaxMaxRecorder", training=False)
    assert bits_equal(to_np(y), to_np(base)) and to_np(M)[0] == 7.0
    with pytest.raises(K.KernelError):
        K.range_recorder(base, None, M, 9)
    with pytest.raises(K.KernelError):
        K.range_recorder(base, None, M, "MinMaxMinMaxRecorder")      # the minimum array is missing


def test_recorder_invariants_at_benchmark_size(dev):
    """Properties that hold whatever the data: running extrema equal the extrema of everything seen (and of the
    starting zero); a moving average fed a constant batch maximum c follows c (1 - decay^n)."""
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    m, M = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
    A = torch.zeros(1, device=dev)
    lo, hi, amax = 0.0, 0.0, 0.0
    for it in range(3):
        x = torch.randn((256, 65536), device=dev, generator=g) * (1 + it)
        y = K.range_recorder(x, m, M, "MinMaxMinMaxRecorder")
        K.range_recorder(x, None, A, "AbsMaxRecorder", y=x)
        assert torch.equal(y, x)
        lo, hi, amax = min(lo, x.min().item()), max(hi, x.max().item()), max(amax, x.abs().max().item())
        assert (m.item(), M.item(), A.item()) == (lo, hi, amax)
    x = torch.rand((64, 4096), device=dev, generator=g)
    x[17, 33] = 5.0
    V = torch.zeros(1, device=dev)
    for n in range(1, 40):
        K.range_recorder(x, None, V, "MaxMvaRecorder", decay=0.9, y=x)
        assert abs(V.item() - 5.0 * (1 - 0.9 ** n)) < 5e-6 * n
    lo_v, hi_v = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
    x[3, 5] = -2.0
    for n in range(1, 20):
        K.range_recorder(x, lo_v, hi_v, "MinMaxMvaRecorder", decay=0.75, y=x)
        assert abs(lo_v.item() + 2.0 * (1 - 0.75 ** n)) < 5e-6 * n and abs(hi_v.item() - 5.0 * (1 - 0.75 ** n)) < 5e-6 * n


# ------------------------------------------------------------------------------------- functions through the registry
def test_recorder_functions_forward_backward(ctx):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    for kind, call in (("MinMaxMinMaxRecorder", qnn.minmax_minmax_recorder), ("AbsMaxRecorder", qnn.abs_max_recorder),
                       ("MinMaxMvaRecorder", qnn.minmax_mva_recorder), ("MaxMaxRecorder", qnn.max_max_recorder),
                       ("MaxMvaRecorder", qnn.max_mva_recorder)):
        two = kind.startswith("MinMax")
        xv = _var(x)
        xv.need_grad = True
        stats = [_var(np.zeros((1, 1, 1), np.float32)) for _ in range(2 if two else 1)]
        y = call(xv, *stats)
        assert y.parent.info.type_name == kind
        m_ref, M_ref = np.float32(0), np.float32(0)
        for _ in range(2):
            y.forward()
            m_ref, M_ref = oracle.range_recorder(x, m_ref if two else None, M_ref, kind, 0.99)
        assert bits_equal(y.d, x)
        assert bits_equal(stats[-1].d, np.full((1, 1, 1), M_ref))
        if two:
            assert bits_equal(stats[0].d, np.full((1, 1, 1), m_ref))
        # the gradient passes through; accumulated onto a leaf's existing gradient
        dy = rng.standard_normal(x.shape).astype(np.float32)
        xv.g = np.ones_like(x)
        y.backward(dy)
        assert bits_equal(xv.g, dy + 1)
        # training=False: identity, statistics untouched
        frozen = call(xv, *stats, training=False)
        before = [s.d.copy() for s in stats]
        frozen.forward()
        assert bits_equal(frozen.d, x) and all(bits_equal(s.d, b) for s, b in zip(stats, before))


def test_sink(ctx):
    a, b = _var(np.ones((2, 3), np.float32)), _var(np.ones((4,), np.float32))
    a.need_grad = b.need_grad = True
    h = F.relu(a)
    end = F.sink(h, b)
    end.forward()
    a.g, b.g = 0, 0
    end.backward(None)
    assert np.array_equal(b.g, np.ones(4, np.float32)) and np.array_equal(a.g, np.ones((2, 3), np.float32))


# ------------------------------------------------------------------------------------------------ converted graphs
def small_net(x):
    h = F.relu(PF.convolution(x, 8, (3, 3), pad=(1, 1), name='c1'))
    h = F.relu(PF.convolution(h, 8, (3, 3), stride=(2, 2), name='c2'))
    h = F.relu(PF.affine(h, 32, name='f1'))
    return PF.affine(h, 10, name='f2')


def randomise_parameters(rng):
    for k, v in nn.get_parameters(grad_only=False).items():
        v.d = (rng.standard_normal(v.shape) * (0.2 if k.endswith('W') else 0.05)).astype(np.float32)


def oracle_training_graph(x, cfg):
    """small_net's simulated-quantization graph computed with the oracle: D -> function -> Q along the chain, weights
    and biases through Q -> D, scales read from the registered parameters."""
    rm, nr = cfg.round_mode, cfg.narrow_range
    P = {k: v.d for k, v in nn.get_parameters(grad_only=False).items()}

    def sz(scope, name, nd):
        return P['%s/scale-%s' % (scope, name)].reshape((1,) * nd), P['%s/zeropoint-%s' % (scope, name)].reshape((1,) * nd)

    def qdq(v, scope, name):
        s, z = sz(scope, name, v.ndim)
        q, z2 = oracle.quantize_linear(v, s, z, rm, nr, 1)
        return oracle.dequantize_linear(q, s, z2)

    h = oracle.convolution(x, P['c1/conv/W'], P['c1/conv/b'], pad=(1, 1))
    h = np.maximum(qdq(h, 'ReLU-1', 'x0'), 0)
    h = qdq(h, 'Convolution-2', 'x0')
    h = oracle.convolution(h, qdq(P['c2/conv/W'], 'Convolution-2', 'w0'), qdq(P['c2/conv/b'], 'Convolution-2', 'b'),
                           stride=(2, 2))
    h = np.maximum(qdq(h, 'ReLU-3', 'x0'), 0)
    h = qdq(h, 'Affine-4', 'x0')
    h = oracle.affine(h.reshape(h.shape[0], -1), qdq(P['f1/affine/W'], 'Affine-4', 'w0'),
                      qdq(P['f1/affine/b'], 'Affine-4', 'b'))
    h = np.maximum(qdq(h, 'ReLU-5', 'x0'), 0)
    return oracle.affine(h, P['f2/affine/W'], P['f2/affine/b'])


def check_every_function(y):
    """Each function of y's graph against the oracle fed the inputs the device function read: the quantize /
    dequantize / ReLU / recorder steps bit for bit, the products within the acceptance tolerance."""
    counts = {}

    def check(f):
        t = f.info.type_name
        ins = [i.d for i in f.inputs]
        out = f.outputs[0].d
        a = f.info.args
        if t == 'Convolution':
            want = oracle.convolution(ins[0], ins[1], ins[2] if len(ins) > 2 else None, pad=a['pad'],
                                      stride=a['stride'], dilation=a['dilation'], group=a['group'])
            assert max_rel_err(out, want) < TOL, (t, max_rel_err(out, want))
        elif t == 'Affine':
            want = oracle.affine(ins[0].reshape(ins[0].shape[0], -1), ins[1], ins[2] if len(ins) > 2 else None)
            assert max_rel_err(out, want) < TOL, (t, max_rel_err(out, want))
        elif t == 'ReLU':
            assert bits_equal(out, np.maximum(ins[0], 0))
        elif t == 'QuantizeLinear':
            want, _ = oracle.quantize_linear(ins[0], ins[1], ins[2], a['round_mode'], a['narrow_range'], a['dtype'])
            assert bits_equal(out, want), (t, first_mismatch(out, want))
            assert np.array_equal(out, np.round(out)) and out.min() >= -128 and out.max() <= 127
        elif t == 'DequantizeLinear':
            want = oracle.dequantize_linear(ins[0], ins[1], ins[2])
            assert bits_equal(out, want), (t, first_mismatch(out, want))
        elif t.endswith('Recorder'):
            assert bits_equal(out, ins[0])
        else:
            raise AssertionError("unexpected function %s" % t)
        counts[t] = counts.get(t, 0) + 1
    y.visit(check)
    return counts


def test_scheduler_end_to_end(ctx):
    rng = np.random.default_rng(2024)
    x = nn.Variable((16, 3, 16, 16))
    y = small_net(x)
    randomise_parameters(rng)
    float_net = GC.GraphConverter([GC.FunctionModifier()]).convert(y)      # an untouched copy to compare with
    float_in = float_net
    while float_in.parent is not None:
        float_in = float_in.parent.inputs[0]
    cfg = QATConfig()
    # the activation recorders average from zero with decay 0.99: they need a few hundred batches to settle
    n_rec = 400
    cfg.niter_to_recording, cfg.niter_to_training = 1, 1 + n_rec
    sched = QATScheduler(cfg)
    sched(y)

    batches = [rng.standard_normal(x.shape).astype(np.float32) * (1 + 0.1 * (i % 5)) for i in range(n_rec + 3)]
    seen_max = {}
    for i, data in enumerate(batches):
        sched.step()
        x.d = data
        float_in.d = data
        y.forward()
        float_net.forward()
        if sched.state != QNNState.TRAINING and i < 8:
            # the recorders are identity functions: the recording graph computes what the float graph computes
            assert bits_equal(y.d, float_net.d), (i, first_mismatch(y.d, float_net.d))
        if sched.state == QNNState.RECORDING and i < 5:
            seen_max[i] = nn.get_parameter('Affine-4/M-w0').d.ravel()[0]
            if i == 2:
                assert check_every_function(y) == {'Convolution': 2, 'Affine': 2, 'ReLU': 3, 'MaxMvaRecorder': 5,
                                                   'MinMaxMinMaxRecorder': 4}
    assert sched.state == QNNState.TRAINING
    # weights did not change while recording: their running maximum is the weight maximum from the first batch on
    W = nn.get_parameter('f1/affine/W').d
    assert all(v == W.max() for v in seen_max.values()) and len(seen_max) == 4
    assert nn.get_parameter('Affine-4/m-w0').d.ravel()[0] == W.min()
    # the activation statistic of four recorded batches is the moving average of their maxima, from zero
    h = np.maximum(oracle.convolution(batches[1], nn.get_parameter('c1/conv/W').d, nn.get_parameter('c1/conv/b').d,
                                      pad=(1, 1)), 0)
    first = np.float32(np.float32(1.0 - 0.99) * h.max())
    settled = nn.get_parameter('Convolution-2/M-x0').d.ravel()[0]
    assert first < settled < 1.5 * h.max() and settled > 0.5 * h.max()

    # the simulated-quantization graph, function by function, against the oracle
    counts = check_every_function(y)
    assert counts == {'Convolution': 2, 'Affine': 2, 'ReLU': 3, 'QuantizeLinear': 9, 'DequantizeLinear': 9}
    # and as a whole against the same chain computed on the oracle alone; a value that sits on a rounding boundary
    # may fall to the other side there, which moves it by one quantization step
    want = oracle_training_graph(batches[-1], cfg)
    got = y.d
    assert got.shape == want.shape == (16, 10)
    assert max_rel_err(got, want) < 0.05, max_rel_err(got, want)
    # and it is a quantized network: close to the float one, not equal to it
    err = max_rel_err(got, float_net.d)
    assert 0 < err < 0.3, err

    # gradients flow through the Q / DQ pairs (straight-through: dy / scale * scale)
    for v in nn.get_parameters().values():
        v.g = 0
    y.backward(np.ones((16, 10), np.float32))
    gW = nn.get_parameter('f1/affine/W').g
    relu5 = y.parent.inputs[0]
    dpre = (relu5.d > 0).astype(np.float32) * (np.ones((16, 10), np.float32) @ nn.get_parameter('f2/affine/W').d.T)
    h_in = y.parent.inputs[0].parent.inputs[0].parent.inputs[0].parent.inputs[0].parent.inputs[0]   # Affine-4's input
    assert h_in.parent.info.type_name == 'DequantizeLinear'
    want_gW = h_in.d.reshape(16, -1).astype(np.float64).T @ dpre.astype(np.float64)
    assert max_rel_err(gW, want_gW) < 1e-3, max_rel_err(gW, want_gW)
    assert np.abs(nn.get_parameter('c1/conv/W').g).max() > 0


@pytest.mark.parametrize("name", ["sub2", "mul2", "div2"])
def test_two_input_arithmetic_functions(ctx, name):
    """Sub2, Mul2, Div2 (sub2.hpp:41, mul2.hpp:42, div2.hpp:44) through the registry: fp32 results bit for bit (one
    IEEE operation per element), and the gradients of base_transform_binary.hpp:286-336 -- dy, -dy | dy * x1, dy * x0 |
    dy / x1, -dy * x0 / (x1 * x1), each operation rounded on its own -- overwritten and accumulated."""
    rng = np.random.default_rng(23)
    shape = (5, 7, 9)                                           # 315 elements: a vector part and a tail
    a = rng.standard_normal(shape).astype(np.float32)
    b = (rng.standard_normal(shape) + np.float32(3.0) * rng.choice([-1, 1], shape)).astype(np.float32)
    a.ravel()[:3] = [0.0, -0.0, np.inf]
    f32 = np.float32
    with np.errstate(all="ignore"):
        fwd = {"sub2": a - b, "mul2": a * b, "div2": a / b}[name]
        g = rng.standard_normal(shape).astype(np.float32)
        g0 = {"sub2": g, "mul2": g * b, "div2": g / b}[name]
        g1 = {"sub2": -g, "mul2": g * a, "div2": (-g * a) / (b * b)}[name]
    va, vb = _var(a), _var(b)
    va.need_grad = vb.need_grad = True
    y = getattr(F, name)(va, vb)
    y.forward()
    assert bits_equal(y.d, fwd.astype(f32))
    va.g, vb.g = 0.0, 0.0
    y.backward(g)
    with np.errstate(all="ignore"):
        assert bits_equal(va.g, (f32(0) + g0).astype(f32)) and bits_equal(vb.g, (f32(0) + g1).astype(f32))
    # one variable on both sides: its gradient is the sum of the two (x - x, x * x, x / x)
    vc = _var(b)
    vc.need_grad = True
    z = getattr(F, name)(vc, vc)
    z.forward()
    vc.g = 0.0
    z.backward(g)
    with np.errstate(all="ignore"):
        h0 = {"sub2": g, "mul2": g * b, "div2": g / b}[name]
        h1 = {"sub2": -g, "mul2": g * b, "div2": (-g * b) / (b * b)}[name]
        assert bits_equal(vc.g, ((f32(0) + h0) + h1).astype(f32))
    # inputs that broadcast against each other (utils/base_transform_binary.hpp:58-86), against the oracle
    c = (rng.standard_normal((5, 1, 9)) + np.float32(3.0)).astype(np.float32)
    vd = _var(c)
    vd.need_grad = True
    w = getattr(F, name)(va, vd)
    assert w.shape == shape
    w.forward()
    assert bits_equal(w.d, oracle.transform_binary(name, a, c))
    va.g, vd.g = 0.0, 0.0
    w.backward(g)
    with np.errstate(all="ignore"):
        assert bits_equal(va.g, oracle.transform_binary_backward(name, 0, g, a, c))
        ref1 = oracle.transform_binary_backward(name, 1, g, a, c)
    fin = np.isfinite(ref1)
    assert np.array_equal(np.isfinite(vd.g), fin) and np.allclose(vd.g[fin], ref1[fin], rtol=1e-5, atol=1e-5)
    with pytest.raises(RuntimeError):
        getattr(F, name)(va, _var(np.zeros((5, 2, 9), np.float32)))     # 7 against 2: not a broadcast


def test_add2_and_concatenate_functions(ctx):
    """add2.cpp:39-77 and concatenate.cpp:62-104 through the registry: forward values, gradients written and
    accumulated, shape checks."""
    rng = np.random.default_rng(11)
    a, b = rng.standard_normal((3, 4, 5)).astype(np.float32), rng.standard_normal((3, 4, 5)).astype(np.float32)
    va, vb = _var(a), _var(b)
    va.need_grad = vb.need_grad = True
    y = F.add2(va, vb)
    y.forward()
    assert bits_equal(y.d, a + b)
    g = rng.standard_normal((3, 4, 5)).astype(np.float32)
    va.g, vb.g = 1.5, 0.0
    y.backward(g)
    assert bits_equal(vb.g, g)
    assert np.allclose(va.g, g) or np.allclose(va.g, g + 1.5)      # written, or added when the graph accumulates
    # the broadcasting fall-back of add2.cpp:28-37
    c = rng.standard_normal((3, 1, 5)).astype(np.float32)
    vc = _var(c)
    vc.need_grad = True
    z = F.add2(va, vc)
    assert z.shape == (3, 4, 5)
    z.forward()
    assert bits_equal(z.d, a + c)
    va.g, vc.g = 0.0, 0.0
    z.backward(g)
    assert bits_equal(va.g, (np.float32(0) + g).astype(np.float32))
    assert np.allclose(vc.g, g.sum(1, keepdims=True), rtol=1e-6, atol=1e-6)
    with pytest.raises(RuntimeError):
        F.add2(va, _var(np.zeros((3, 2, 5), np.float32)))          # 4 against 2: not a broadcast

    parts = [rng.standard_normal((2, n, 3, 7)).astype(np.float32) for n in (4, 1, 6)]
    vs = [_var(p) for p in parts]
    for v in vs:
        v.need_grad = True
    for axis in (1, -3):
        c = F.concatenate(*vs, axis=axis)
        assert c.shape == (2, 11, 3, 7)
        c.forward()
        assert bits_equal(c.d, np.concatenate(parts, axis=1))
        gc_ = rng.standard_normal(c.shape).astype(np.float32)
        for v in vs:
            v.g = 0
        c.backward(gc_)
        off = 0
        for v, p in zip(vs, parts):
            assert bits_equal(v.g, gc_[:, off:off + p.shape[1]])
            off += p.shape[1]
    last = F.concatenate(_var(np.ones((2, 3), np.float32)), _var(np.zeros((2, 2), np.float32)))    # default: last axis
    last.forward()
    assert last.d.tolist() == [[1, 1, 1, 0, 0], [1, 1, 1, 0, 0]]
    with pytest.raises(RuntimeError):
        F.concatenate(vs[0], _var(np.zeros((2, 4, 3, 8), np.float32)), axis=1)


def test_two_views_of_one_gradient_accumulate(ctx):
    """A variable and a view of it (same arrays) feeding one function: the second contribution to the shared gradient
    is added to the first, not written over it."""
    rng = np.random.default_rng(3)
    x = _var(rng.standard_normal((4, 6)).astype(np.float32))
    x.need_grad = True
    h = F.relu(x)
    y = F.add2(h, h.reshape(h.shape))
    y.forward()
    g = rng.standard_normal((4, 6)).astype(np.float32)
    x.g = 0
    y.backward(g)
    assert bits_equal(x.g, np.where(x.d > 0, 2 * g, 0).astype(np.float32))


def residual_concat_net(x):
    h = F.relu(PF.convolution(x, 4, (3, 3), pad=(1, 1), name='c1'))
    r = F.relu(PF.convolution(h, 4, (3, 3), pad=(1, 1), name='c2'))
    s = F.add2(h, r)
    t = F.relu(PF.convolution(s, 3, (3, 3), pad=(1, 1), name='c3'))
    return PF.affine(F.concatenate(t, s, axis=1), 6, name='f')


def test_scheduler_with_add2_and_concatenate(ctx):
    """A residual / concatenating network through the three states: the recording graph computes the float values,
    and in the training graph the inputs of Add2 and of Concatenate sit on one quantization grid each."""
    rng = np.random.default_rng(8)
    x = nn.Variable((4, 3, 8, 8))
    y = residual_concat_net(x)
    randomise_parameters(rng)
    float_net = GC.GraphConverter([GC.FunctionModifier()]).convert(y)
    float_in = float_net
    while float_in.parent is not None:
        float_in = float_in.parent.inputs[0]
    cfg = QATConfig()
    cfg.niter_to_recording, cfg.niter_to_training = 1, 60
    sched = QATScheduler(cfg)
    sched(y)
    for i in range(62):
        sched.step()
        data = rng.standard_normal(x.shape).astype(np.float32)
        x.d = data
        float_in.d = data
        y.forward()
        float_net.forward()
        if sched.state == QNNState.RECORDING and i < 4:
            assert bits_equal(y.d, float_net.d)
    assert sched.state == QNNState.TRAINING
    fs = []
    y.visit(fs.append)
    for kind in ('Add2', 'Concatenate'):
        f = [g for g in fs if g.info.type_name == kind][0]
        dq = [v.parent for v in f.inputs]
        assert all(g.info.type_name == 'DequantizeLinear' for g in dq)
        scale = float(dq[0].inputs[1].d.ravel()[0])
        assert all(g.inputs[1] is dq[0].inputs[1] for g in dq) and scale > 0
        for v in f.inputs:                   # every input value is a whole number of steps of the shared scale
            steps = v.d / np.float32(scale)
            assert np.abs(steps - np.round(steps)).max() < 1e-3
    err = max_rel_err(y.d, float_net.d)
    assert 0 < err < 0.5, err
    y.backward(np.ones(y.shape, np.float32))
    assert np.abs(nn.get_parameter('c1/conv/W').g).max() > 0


def test_add2_and_concatenate_saved_and_reloaded(ctx, tmp_path):
    from nnabla_amd.utils.nnp_graph import NnpLoader
    from nnabla_amd.utils.save import save
    from test_nnp_save import contents_of
    x = nn.Variable((3, 3, 8, 8))
    y = residual_concat_net(x)
    randomise_parameters(np.random.default_rng(21))
    path = str(tmp_path / 'res.nnp')
    save(path, contents_of(x, y, 3))
    data = np.random.default_rng(22).standard_normal(x.shape).astype(np.float32)
    x.d = data
    y.forward()
    ex = NnpLoader(path).get_executor('runtime')
    ex.data_variables['x'].d = data
    ex.execute()
    assert bits_equal(ex.output_variables['y'].d, y.d)


def test_recording_with_other_recorders_matches_oracle(ctx):
    """MinMaxMva activations / AbsMax weights on an MLP: every registered statistic against the oracle's recorders fed
    the same tensors."""
    rng = np.random.default_rng(77)
    x = nn.Variable((32, 64))
    h = F.relu(PF.affine(x, 48, name='a'))
    y = PF.affine(F.relu(PF.affine(h, 40, name='b')), 8, name='c')
    randomise_parameters(rng)
    cfg = QATConfig()
    cfg.skip_inputs_layers, cfg.skip_outputs_layers = [], []
    cfg.record_layers = ['Affine']
    cfg.recorder_activation = qnn.MinMaxMvaRecorderCallback
    cfg.recorder_weight = qnn.AbsMaxRecorderCallback
    ranks = FunctionsRankRecorder()
    y.visit(ranks)
    y_rec = GC.GraphConverter([GC.QuantizeNonQNNToRecordingModifier(ranks.functions_ranks, config=cfg)]).convert(y)
    x_rec = y_rec
    while x_rec.parent is not None:
        x_rec = x_rec.parent.inputs[0]
    P = {k: v.d for k, v in nn.get_parameters(grad_only=False).items()}
    ref = {}
    for it in range(3):
        data = rng.standard_normal(x.shape).astype(np.float32) * (it + 1)
        x_rec.d = data
        y_rec.forward()
        acts = {'Affine-0': data}
        acts['Affine-2'] = np.maximum(oracle.affine(data, P['a/affine/W'], P['a/affine/b']), 0)
        acts['Affine-4'] = np.maximum(oracle.affine(acts['Affine-2'], P['b/affine/W'], P['b/affine/b']), 0)
        for scope, pre in (('Affine-0', 'a'), ('Affine-2', 'b'), ('Affine-4', 'c')):
            act = to_np_device(y_rec, scope)
            lo, hi = ref.get(scope + 'x', (np.float32(0), np.float32(0)))
            # the recorded activation is the device's own (its fp32 sums differ from the oracle's in the last bits)
            ref[scope + 'x'] = oracle.range_recorder(act, lo, hi, 'MinMaxMvaRecorder', 0.99)
            assert max_rel_err(act, acts[scope]) < TOL
            for j, leaf in enumerate(('W', 'b')):
                _, Mw = oracle.range_recorder(P['%s/affine/%s' % (pre, leaf)], None,
                                              ref.get(scope + leaf, np.float32(0)), 'AbsMaxRecorder')
                ref[scope + leaf] = Mw
                assert nn.get_parameter('%s/M-w%d' % (scope, j)).d.ravel()[0] == Mw
            assert bits_equal(nn.get_parameter(scope + '/m-x0').d.ravel(), [ref[scope + 'x'][0]])
            assert bits_equal(nn.get_parameter(scope + '/M-x0').d.ravel(), [ref[scope + 'x'][1]])


def to_np_device(y_rec, scope):
    """The tensor that entered the activation recorder registered under ``scope`` in the graph of ``y_rec``."""
    target = nn.get_parameter(scope + '/M-x0')
    found = []

    def look(f):
        if f.info.type_name == 'MinMaxMvaRecorder' and f.inputs[2] is target:
            found.append(f.inputs[0].d)
    y_rec.visit(look)
    assert len(found) == 1
    return found[0]


# ------------------------------------------------------------------------------------------------- saving as NNP
def test_scheduler_save_and_reload(ctx, tmp_path):
    """The evaluation network of a finished schedule written with QATScheduler.save, read back with NnpLoader and
    executed: the same bits as the graph it was written from."""
    from nnabla_amd.utils.nnp_graph import NnpLoader
    rng = np.random.default_rng(5)
    x = nn.Variable((8, 3, 16, 16))
    y = small_net(x)
    randomise_parameters(rng)
    vx = nn.Variable((4, 3, 16, 16))
    vy = small_net(vx)                                  # shares the parameters
    cfg = QATConfig()
    cfg.recorder_activation = qnn.MaxMaxRecorderCallback
    cfg.niter_to_recording, cfg.niter_to_training = 0, 3
    sched = QATScheduler(cfg)
    sched(y)
    sched(vy, training=False)
    for i in range(5):
        sched.step()
        x.d = rng.standard_normal(x.shape).astype(np.float32)
        y.forward()
    assert sched.state == QNNState.TRAINING
    data = rng.standard_normal(vx.shape).astype(np.float32)
    vx.d = data
    vy.forward()
    counts = check_every_function(vy)
    assert counts['QuantizeLinear'] == 9

    path = str(tmp_path / 'qnn.nnp')
    sched.save(path, vx, batch_size=4)
    loader = NnpLoader(path)
    ex = loader.get_executor('runtime')
    assert list(ex.data_variables) == ['x0'] and list(ex.output_variables) == ['y0']
    ex.data_variables['x0'].d = data
    ex.execute()
    assert bits_equal(ex.output_variables['y0'].d, vy.d), first_mismatch(ex.output_variables['y0'].d, vy.d)
    names = []
    ex.output_variables['y0'].visit(lambda f: names.append(f.info.type_name))
    mine = []
    vy.visit(lambda f: mine.append(f.info.type_name))
    assert names == mine
    assert np.array_equal(loader.get_parameters()['ReLU-1/scale-x0'].d, nn.get_parameter('ReLU-1/scale-x0').d)
    with pytest.raises(NotImplementedError):
        sched.save(path, vx, deploy=True)


def test_every_function_saved_and_reloaded(ctx, tmp_path):
    from nnabla_amd.utils.nnp_graph import NnpLoader
    from nnabla_amd.utils.save import save
    from test_nnp_save import contents_of, every_function_net
    x = nn.Variable((6, 3, 6, 6))
    y = every_function_net(x)
    for k, v in nn.get_parameters(grad_only=False).items():
        if k in ('mmq/ql_min', 'ql/z'):
            v.d = 0
        elif k == 'mmq/ql_max':
            v.d = 255
        elif k == 'ql/s':
            v.d = 0.05
    path = str(tmp_path / 'all.nnp')
    save(path, contents_of(x, y, 6))                   # before any forward: INQ / min-max state as initialised
    data = np.random.default_rng(1).standard_normal(x.shape).astype(np.float32)
    x.d = data
    y.forward()
    ex = NnpLoader(path).get_executor('runtime')
    ex.data_variables['x'].d = data
    ex.execute()
    assert bits_equal(ex.output_variables['y'].d, y.d), first_mismatch(ex.output_variables['y'].d, y.d)
