"""Graphs loaded from NNP archives run on the hip:float classes: every function's output is checked against the CPU
oracle applied to that function's own (GPU-produced) inputs, so a quantizer tie cannot make the two chains drift."""
import numpy as np
import pytest

import nnabla_amd as nn
import oracle
from nnabla_amd.ext_utils import get_extension_context
from nnabla_amd.utils.nnp_graph import NnpLoader, save_nnp
from util import bits_equal, max_rel_err

pytestmark = pytest.mark.gpu
TIGHT = 5e-6


@pytest.fixture()
def ctx(dev):
    c = get_extension_context('hip', device_id='0')
    with nn.context_scope(c):
        yield c


def _var(name, kind, shape):
    return 'variable { name: "%s" type: "%s" shape: { %s } }\n' % (name, kind, " ".join("dim: %d" % d for d in shape))


def _fn(name, ftype, ins, out, param=""):
    return 'function { name: "%s" type: "%s" %s output: "%s" %s }\n' % (
        name, ftype, " ".join('input: "%s"' % i for i in ins), out, param)


MLP = ('network {\n name: "mlp"\n batch_size: 16\n'
       + _var("x", "Buffer", (-1, 32))
       + "".join(_var(n, "Parameter", s) for n, s in [
           ("fc0/W", (32, 48)), ("fc0/I", (32, 48)), ("fc0/b", (48,)), ("fc1/W", (48, 40)), ("fc1/Wb", (48, 40)),
           ("fc1/alpha", (40,)), ("fc1/b", (40,)), ("mm/qr_min", (1, 1)), ("mm/qr_max", (1, 1)), ("mm/ql_min", (1, 1)),
           ("mm/ql_max", (1, 1)), ("fc2/W", (40, 10)), ("fc2/Wb", (40, 10))])
       + _fn("q0", "FixedPointQuantize", ["x"], "h0", "fixed_point_quantize_param { sign: true n: 6 delta: 0.125 }")
       + _fn("fc0", "INQAffine", ["h0", "fc0/W", "fc0/I", "fc0/b"], "h1",
             'inq_affine_param { base_axis: 1 num_bits: 4 inq_iterations: 0 selection_algorithm: "largest_abs" seed: -1 }')
       + _fn("r1", "ReLU", ["h1"], "h2")
       + _fn("q1", "Pow2Quantize", ["h2"], "h3", "pow2_quantize_param { sign: false with_zero: true n: 4 m: 2 }")
       + _fn("fc1", "BinaryWeightAffine", ["h3", "fc1/W", "fc1/Wb", "fc1/alpha", "fc1/b"], "h4",
             "binary_weight_affine_param { base_axis: 1 quantize_zero_to: -1.0 }")
       + _fn("q2", "MinMaxQuantize", ["h4", "mm/qr_min", "mm/qr_max", "mm/ql_min", "mm/ql_max"], "h5",
             "min_max_quantize_param { decay: 0.9 x_min_max: true ema: true ste_fine_grained: true eps: 0.01 }")
       + _fn("fc2", "BinaryConnectAffine", ["h5", "fc2/W", "fc2/Wb"], "y", "binary_connect_affine_param { base_axis: 1 }")
       + '}\nexecutor { name: "infer" network_name: "mlp" data_variable { variable_name: "x" data_name: "x" } '
         'output_variable { variable_name: "y" data_name: "y" } }\n')


def test_quantized_mlp_from_nnp(ctx, tmp_path):
    rng = np.random.RandomState(5)
    params = {
        "fc0/W": (rng.randn(32, 48) * 0.1).astype(np.float32), "fc0/I": (np.zeros((32, 48), np.float32), False),
        "fc0/b": rng.randn(48).astype(np.float32), "fc1/W": (rng.randn(48, 40) * 0.1).astype(np.float32),
        "fc1/Wb": np.zeros((48, 40), np.float32), "fc1/alpha": np.zeros(40, np.float32),
        "fc1/b": rng.randn(40).astype(np.float32), "mm/qr_min": np.float32([[-1.0]]), "mm/qr_max": np.float32([[1.0]]),
        "mm/ql_min": np.float32([[0.0]]), "mm/ql_max": np.float32([[255.0]]),
        "fc2/W": (rng.randn(40, 10) * 0.1).astype(np.float32), "fc2/Wb": np.zeros((40, 10), np.float32)}
    params["fc1/W"].ravel()[:5] = 0.0
    path = str(tmp_path / "mlp.nnp")
    save_nnp(path, MLP, params)
    exe = NnpLoader(path).get_executor("infer")
    v = exe.network.variables
    x = (rng.randn(16, 32) * 2).astype(np.float32)
    exe.data_variables["x"].d = x
    exe.execute()

    assert bits_equal(v["h0"].d, oracle.fixed_point_quantize(x, True, 6, 0.125))
    inq = oracle.Inq(32 * 48, 4, (0,), "largest_abs")
    Wc, Ic = params["fc0/W"].copy(), np.zeros((32, 48), np.int32)
    ref_h1 = inq.affine(v["h0"].d, Wc, Ic, params["fc0/b"])
    assert bits_equal(v["fc0/W"].d, Wc) and np.array_equal(v["fc0/I"].d, Ic) and v["fc0/I"].d.dtype == np.int32
    assert max_rel_err(v["h1"].d, ref_h1) <= TIGHT
    assert bits_equal(v["h2"].d, np.maximum(v["h1"].d, 0))
    assert bits_equal(v["h3"].d, oracle.pow2_quantize(v["h2"].d, False, True, 4, 2))
    ref_h4, ref_wb, ref_alpha = oracle.binary_weight_affine(v["h3"].d, params["fc1/W"], params["fc1/b"], -1.0)
    assert bits_equal(v["fc1/Wb"].d, ref_wb) and (v["fc1/Wb"].d.ravel()[:5] == -1).all()
    np.testing.assert_allclose(v["fc1/alpha"].d, ref_alpha, rtol=2e-6)
    assert max_rel_err(v["h4"].d, ref_h4) <= TIGHT
    ref_h5, ref_min, ref_max, _ = oracle.min_max_quantize(v["h4"].d, params["mm/qr_min"], params["mm/qr_max"],
                                                       params["mm/ql_min"], params["mm/ql_max"], 0.9, True, True, 0.01)
    assert bits_equal(v["h5"].d, ref_h5)
    assert bits_equal(v["mm/qr_min"].d, ref_min) and bits_equal(v["mm/qr_max"].d, ref_max)   # state lives in the params
    ref_y, ref_wb2 = oracle.binary_connect_affine(v["h5"].d, params["fc2/W"], None, 1.0)
    assert bits_equal(v["fc2/Wb"].d, ref_wb2) and max_rel_err(exe.output_variables["y"].d, ref_y) <= TIGHT


CNN = ('network {\n name: "cnn"\n batch_size: 2\n'
       + _var("x", "Buffer", (-1, 4, 10, 10))
       + "".join(_var(n, "Parameter", s) for n, s in [
           ("c0/W", (8, 4, 3, 3)), ("c0/Wb", (8, 4, 3, 3)), ("c0/alpha", (8,)), ("c0/b", (8,)),
           ("c1/W", (6, 4, 3, 3)), ("c1/Wb", (6, 4, 3, 3)), ("c2/W", (5, 6, 2, 2)), ("c2/I", (5, 6, 2, 2)),
           ("fc/W", (5 * 4 * 4, 3)), ("fc/b", (3,))])
       + _fn("c0", "BinaryWeightConvolution", ["x", "c0/W", "c0/Wb", "c0/alpha", "c0/b"], "h0",
             "binary_weight_convolution_param { base_axis: 1 pad: { dim: 1 dim: 1 } stride: { dim: 1 dim: 1 } "
             "dilation: { dim: 1 dim: 1 } group: 1 quantize_zero_to: 1.0 }")
       + _fn("r0", "ReLU", ["h0"], "h1", "relu_param { inplace: false }")
       + _fn("c1", "BinaryConnectConvolution", ["h1", "c1/W", "c1/Wb"], "h2",
             "binary_connect_convolution_param { base_axis: 1 pad: { dim: 1 dim: 1 } stride: { dim: 2 dim: 2 } group: 2 }")
       + _fn("c2", "INQConvolution", ["h2", "c2/W", "c2/I"], "h3",
             'inq_convolution_param { base_axis: 1 num_bits: 3 inq_iterations: 0 selection_algorithm: "largest_abs" }')
       + _fn("fc", "Affine", ["h3", "fc/W", "fc/b"], "y", "affine_param { base_axis: 1 }")
       + "}\n")


def test_quantized_cnn_from_nnp(ctx, tmp_path):
    rng = np.random.RandomState(6)
    shapes = {"c0/W": (8, 4, 3, 3), "c0/b": (8,), "c1/W": (6, 4, 3, 3), "c2/W": (5, 6, 2, 2), "fc/W": (80, 3),
              "fc/b": (3,)}
    params = {k: (rng.randn(*s) * 0.1).astype(np.float32) for k, s in shapes.items()}
    path = str(tmp_path / "cnn.nnp")
    save_nnp(path, CNN, params)
    net = NnpLoader(path).get_network("cnn", batch_size=3)
    v = net.variables
    assert list(net.inputs) == ["x"] and list(net.outputs) == ["y"] and v["y"].shape == (3, 3)
    x = rng.randn(3, 4, 10, 10).astype(np.float32)
    v["x"].d = x
    v["y"].forward()
    ref_h0, ref_wb, ref_alpha = oracle.binary_weight_convolution(x, params["c0/W"], params["c0/b"], (1, 1), (1, 1),
                                                                 (1, 1), 1, 1.0)
    assert bits_equal(v["c0/Wb"].d, ref_wb) and max_rel_err(v["h0"].d, ref_h0) <= TIGHT
    np.testing.assert_allclose(v["c0/alpha"].d, ref_alpha, rtol=2e-6)
    ref_h2, ref_wb1 = oracle.binary_connect_convolution(v["h1"].d, params["c1/W"], None, (1, 1), (2, 2), None, 2, 1.0)
    assert bits_equal(v["c1/Wb"].d, ref_wb1) and max_rel_err(v["h2"].d, ref_h2) <= TIGHT
    inq = oracle.Inq(params["c2/W"].size, 3, (0,), "largest_abs")
    Wc, Ic = params["c2/W"].copy(), np.zeros(params["c2/W"].shape, np.int32)
    ref_h3 = inq.convolution(v["h2"].d, Wc, Ic)
    assert bits_equal(v["c2/W"].d, Wc) and np.array_equal(v["c2/I"].d, Ic)
    assert max_rel_err(v["h3"].d, ref_h3) <= TIGHT
    ref_y = v["h3"].d.reshape(3, -1).astype(np.float64) @ params["fc/W"].astype(np.float64) + params["fc/b"]
    assert max_rel_err(v["y"].d, ref_y) <= TIGHT
    # the loaded graph trains: backward reaches the first layer's weights
    for name in ("c0/W", "c1/W", "c2/W", "fc/W"):
        v[name].zero_grad()
    v["y"].backward(np.ones((3, 3), np.float32))
    assert np.abs(v["c0/W"].g).max() > 0 and np.isfinite(v["c0/W"].g).all()
