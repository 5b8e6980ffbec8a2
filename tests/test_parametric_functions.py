"""Parametric layers: parameter scopes, names, shapes and need_grad flags (CPU: graph construction only), following
the parameter tables of python/src/nnabla/parametric_functions.py (the ``param_desc`` of each layer)."""
import numpy as np
import pytest

import nnabla_amd as nn
import nnabla_amd.parametric_functions as PF
from nnabla_amd.ext_utils import get_extension_context


@pytest.fixture()
def scope():
    nn.clear_parameters()
    with nn.context_scope(get_extension_context('hip', device_id='0')):
        yield
    nn.clear_parameters()


def _flags(grad_only=False):
    return {k: (tuple(v.shape), v.need_grad) for k, v in nn.get_parameters(grad_only=grad_only).items()}


def test_parameter_scope_registry(scope):
    with nn.parameter_scope("a"):
        with nn.parameter_scope("b/c"):
            p = nn.get_parameter_or_create("w", (2, 3), np.arange(6, dtype=np.float32).reshape(2, 3), True)
        q = nn.get_parameter_or_create("b/c/w", (2, 3))
        assert q is p
        frozen = nn.get_parameter_or_create("b/c/w", (2, 3), None, True, as_need_grad=False)
        assert frozen is not p and not frozen.need_grad and np.array_equal(frozen.d, p.d)
    assert list(nn.get_parameters()) == ["a/b/c/w"]
    assert nn.get_parameter("a/b/c/w") is p and nn.get_parameter("a/nope") is None
    with pytest.raises(ValueError):
        nn.get_parameter_or_create("a/b/c/w", (3, 2))
    with pytest.raises(ValueError):
        nn.get_parameter_or_create("fresh", None, None)
    assert nn.pop_parameter("a/b/c/w") is p and not nn.get_parameters()


def test_quantized_layers_register_the_reference_parameters(scope):
    x = nn.Variable((4, 3, 8, 8))
    y = PF.fixed_point_quantized_affine(x, 10, name="fc")
    assert y.shape == (4, 10)
    assert _flags() == {"fc/fp_quantized_affine/W": ((192, 10), True), "fc/fp_quantized_affine/W_q": ((192, 10), False),
                        "fc/fp_quantized_affine/b": ((10,), True), "fc/fp_quantized_affine/b_q": ((10,), False)}
    nn.clear_parameters()
    y = PF.pow2_quantized_convolution(x, 6, (3, 3), pad=(1, 1), quantize_b=False, fix_parameters=True)
    assert y.shape == (4, 6, 8, 8)
    assert _flags() == {"pow2_quantized_conv/W": ((6, 3, 3, 3), True), "pow2_quantized_conv/W_q": ((6, 3, 3, 3), False),
                        "pow2_quantized_conv/b": ((6,), True)}
    assert y.parent.info["type"] == "Convolution"
    # fix_parameters: the graph sees views that do not ask for gradients; the registry keeps need_grad
    assert not any(i.need_grad for i in y.parent.inputs[1].parent.inputs)
    nn.clear_parameters()
    y = PF.min_max_quantized_affine(x, (5, 2), w_min_max=True)
    assert y.shape == (4, 5, 2)
    f = _flags()
    base = "min_max_quantized_affine/"
    assert f[base + "W"] == ((192, 5, 2), True) and f[base + "W_q"] == ((192, 5, 2), False)
    assert f[base + "min_max_quantize_w/min_max_quantize/qr_min"] == ((1, 1, 1), True)
    assert f[base + "min_max_quantize_w/min_max_quantize/ql_max"] == ((1, 1, 1), False)
    assert f[base + "min_max_quantize_b/min_max_quantize/qr_max"] == ((1, 1), True)
    assert nn.get_parameter(base + "min_max_quantize_w/min_max_quantize/qr_max").d.ravel()[0] == 2.0
    assert nn.get_parameter(base + "min_max_quantize_b/min_max_quantize/qr_min").d.ravel()[0] == -6.0
    assert nn.get_parameter(base + "min_max_quantize_b/min_max_quantize/ql_max").d.ravel()[0] == 255.0


def test_binary_inq_and_pruned_layers(scope):
    x = nn.Variable((2, 4, 6, 6))
    PF.binary_connect_affine(x, 7)
    PF.binary_weight_affine(x, 7)
    PF.binary_connect_convolution(x, 5, (3, 3), with_bias=False)
    PF.binary_weight_convolution(x, 6, (3, 3), group=2)
    PF.inq_affine(x, 3, inq_iterations=(10, 20))
    PF.inq_convolution(x, 3, (2, 2))
    PF.pruned_affine(x, 4, rate_w=0.5, prune_b=False)
    PF.pruned_convolution(x, 4, (1, 1))
    PF.affine(x, 2)
    PF.convolution(x, 2, (3, 3), stride=(2, 2))
    f = _flags()
    assert f["bicon_affine/Wb"] == ((144, 7), False) and f["bicon_affine/b"] == ((7,), True)
    assert f["bwn_affine/alpha"] == ((7,), False)
    assert "bicon_conv/b" not in f and f["bicon_conv/W"] == ((5, 4, 3, 3), True)
    assert f["bwn_conv/W"] == ((6, 2, 3, 3), True) and f["bwn_conv/alpha"] == ((6,), False)
    assert f["inq_affine/I"] == ((144, 3), False) and nn.get_parameter("inq_affine/I").d.dtype == np.int32
    assert f["inq_conv/I"] == ((3, 4, 2, 2), False)
    assert f["pruned_affine/W_q"] == ((144, 4), False) and "pruned_affine/b_q" not in f
    assert f["pruned_conv/b_q"] == ((4,), False)
    assert f["affine/W"] == ((144, 2), True) and f["conv/W"] == ((2, 4, 3, 3), True)
    # weights drawn within Glorot's limits from the shared generator
    lim = np.sqrt(6.0 / (144 + 7))
    w = nn.get_parameter("bicon_affine/W").d
    assert np.abs(w).max() <= lim and w.std() > lim / 4
    assert sorted(nn.get_parameters()) == sorted(k for k, v in f.items() if v[1])
