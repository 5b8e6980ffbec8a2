"""``F.*``: the quantization functions (plus affine and relu) with nnabla's signatures
(python/src/nnabla/functions.py:416-691 and the generated function_bases for functions.yaml:6735-7520)."""
from .function import Function


def _n_spatial(x, base_axis):
    base_axis = base_axis if base_axis >= 0 else x.ndim + base_axis
    return x.ndim - (base_axis + 1)


def fixed_point_quantize(x, sign=True, n=8, delta=2 ** -4, quantize=True, ste_fine_grained=True, outputs=None):
    """Fixed-point quantization of ``x`` (returns ``x`` itself when ``quantize`` is False)."""
    if not quantize:
        return x
    f = Function("FixedPointQuantize", None, [int(sign), n, int(ste_fine_grained)], [delta],
                 args=dict(sign=sign, n=n, delta=delta, ste_fine_grained=ste_fine_grained))
    return f(x, outputs=outputs)


def pow2_quantize(x, sign=True, with_zero=True, n=8, m=1, quantize=True, ste_fine_grained=True, outputs=None):
    """Power-of-two quantization of ``x`` (returns ``x`` itself when ``quantize`` is False)."""
    if not quantize:
        return x
    f = Function("Pow2Quantize", None, [int(sign), int(with_zero), n, m, int(ste_fine_grained)],
                 args=dict(sign=sign, with_zero=with_zero, n=n, m=m, ste_fine_grained=ste_fine_grained))
    return f(x, outputs=outputs)


def min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, decay=0.999, x_min_max=False, ema=False,
                     ste_fine_grained=True, eps=0.01, quantize=True, outputs=None):
    """Min-max quantization; ``qr_min`` / ``qr_max`` are updated in place when ``x_min_max`` is set."""
    if not quantize:
        return x
    f = Function("MinMaxQuantize", None, [int(x_min_max), int(ema), int(ste_fine_grained)], [decay, eps],
                 args=dict(decay=decay, x_min_max=x_min_max, ema=ema, ste_fine_grained=ste_fine_grained, eps=eps))
    return f(x, qr_min, qr_max, ql_min, ql_max, outputs=outputs)


def binary_weight_affine(x, weight, binary_weight, alpha, bias=None, base_axis=1, quantize_zero_to=1.0,
                         n_outputs=-1, outputs=None):
    f = Function("BinaryWeightAffine", None, [base_axis], [quantize_zero_to],
                 args=dict(base_axis=base_axis, quantize_zero_to=quantize_zero_to))
    ins = [x, weight, binary_weight, alpha] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def binary_connect_affine(x, weight, binary_weight, bias=None, base_axis=1, quantize_zero_to=1.0, n_outputs=-1,
                          outputs=None):
    f = Function("BinaryConnectAffine", None, [base_axis], [quantize_zero_to],
                 args=dict(base_axis=base_axis, quantize_zero_to=quantize_zero_to))
    ins = [x, weight, binary_weight] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def _conv_iargs(x, base_axis, pad, stride, dilation, group):
    nd = _n_spatial(x, base_axis)
    pad = tuple(pad) if pad is not None else (0,) * nd
    stride = tuple(stride) if stride is not None else (1,) * nd
    dilation = tuple(dilation) if dilation is not None else (1,) * nd
    return nd, list(pad) + list(stride) + list(dilation)


def _conv_args(base_axis, nd, geom, group, **more):
    d = dict(base_axis=base_axis, pad=tuple(geom[:nd]), stride=tuple(geom[nd:2 * nd]),
             dilation=tuple(geom[2 * nd:3 * nd]), group=group)
    d.update(more)
    return d


def binary_weight_convolution(x, weight, binary_weight, alpha, bias=None, base_axis=1, pad=None, stride=None,
                              dilation=None, group=1, quantize_zero_to=1.0, n_outputs=-1, outputs=None):
    nd, geom = _conv_iargs(x, base_axis, pad, stride, dilation, group)
    f = Function("BinaryWeightConvolution", None, [base_axis, group, nd] + geom, [quantize_zero_to],
                 args=_conv_args(base_axis, nd, geom, group, quantize_zero_to=quantize_zero_to))
    ins = [x, weight, binary_weight, alpha] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def binary_connect_convolution(x, weight, binary_weight, bias=None, base_axis=1, pad=None, stride=None,
                               dilation=None, group=1, quantize_zero_to=1.0, n_outputs=-1, outputs=None):
    nd, geom = _conv_iargs(x, base_axis, pad, stride, dilation, group)
    f = Function("BinaryConnectConvolution", None, [base_axis, group, nd] + geom, [quantize_zero_to],
                 args=_conv_args(base_axis, nd, geom, group, quantize_zero_to=quantize_zero_to))
    ins = [x, weight, binary_weight] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def inq_affine(x, weight, indicator_fixedweights, bias=None, base_axis=1, num_bits=4, inq_iterations=(),
               selection_algorithm='largest_abs', seed=-1, n_outputs=-1, outputs=None):
    its = [int(i) for i in inq_iterations]
    f = Function("INQAffine", None, [base_axis, num_bits, seed, len(its)] + its, [], selection_algorithm,
                 args=dict(base_axis=base_axis, num_bits=num_bits, inq_iterations=tuple(its),
                           selection_algorithm=selection_algorithm, seed=seed))
    ins = [x, weight, indicator_fixedweights] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def inq_convolution(x, weight, indicator_fixedweights, bias=None, base_axis=1, pad=None, stride=None, dilation=None,
                    group=1, num_bits=4, inq_iterations=(), selection_algorithm='largest_abs', seed=-1, n_outputs=-1,
                    outputs=None):
    nd, geom = _conv_iargs(x, base_axis, pad, stride, dilation, group)
    its = [int(i) for i in inq_iterations]
    f = Function("INQConvolution", None, [base_axis, group, num_bits, seed, nd] + geom + [len(its)] + its, [],
                 selection_algorithm,
                 args=_conv_args(base_axis, nd, geom, group, num_bits=num_bits, inq_iterations=tuple(its),
                                 selection_algorithm=selection_algorithm, seed=seed))
    ins = [x, weight, indicator_fixedweights] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def affine(x, weight, bias=None, base_axis=1, n_outputs=-1, outputs=None):
    f = Function("Affine", None, [base_axis], args=dict(base_axis=base_axis))
    ins = [x, weight] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def convolution(x, weight, bias=None, base_axis=1, pad=None, stride=None, dilation=None, group=1, channel_last=False,
                n_outputs=-1, outputs=None):
    nd, geom = _conv_iargs(x, base_axis, pad, stride, dilation, group)
    f = Function("Convolution", None, [base_axis, group, int(channel_last), nd] + geom,
                 args=_conv_args(base_axis, nd, geom, group, channel_last=channel_last))
    ins = [x, weight] + ([bias] if bias is not None else [])
    return f(*ins, outputs=outputs)


def relu(x, inplace=False, n_outputs=-1, outputs=None):
    f = Function("ReLU", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x, outputs=outputs)


def add2(x0, x1, inplace=False, n_outputs=-1, outputs=None):
    f = Function("Add2", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x0, x1, n_outputs=n_outputs, outputs=outputs)


def sub2(x0, x1, inplace=False, n_outputs=-1, outputs=None):
    f = Function("Sub2", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x0, x1, n_outputs=n_outputs, outputs=outputs)


def mul2(x0, x1, inplace=False, n_outputs=-1, outputs=None):
    f = Function("Mul2", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x0, x1, n_outputs=n_outputs, outputs=outputs)


def div2(x0, x1, inplace=False, n_outputs=-1, outputs=None):
    f = Function("Div2", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x0, x1, n_outputs=n_outputs, outputs=outputs)


def pow2(x0, x1, inplace=False, n_outputs=-1, outputs=None):
    """Element-wise power x0 ** x1 (not the power-of-two quantizer: that is pow2_quantize)."""
    f = Function("Pow2", None, [int(inplace)], args=dict(inplace=inplace))
    return f(x0, x1, n_outputs=n_outputs, outputs=outputs)


def concatenate(*x, **kw):
    axis = kw.pop('axis', None)
    n_outputs, outputs = kw.pop('n_outputs', -1), kw.pop('outputs', None)
    if axis is None:
        axis = len(x[0].shape) - 1
    f = Function("Concatenate", None, [int(axis)], args=dict(axis=axis))
    return f(*x, n_outputs=n_outputs, outputs=outputs)


def quantize_linear(x, scale, zero_point, round_mode='HALF_AWAY_FROM_ZERO', narrow_range=False, dtype=1,
                    n_outputs=-1, outputs=None):
    """``saturate(round(x / scale) + zero_point)`` to the int8 (``dtype`` 1 or ``numpy.int8``) or uint8 (2 or
    ``numpy.uint8``) range; ``zero_point`` is rounded and saturated in place (functions.yaml:7556-7601)."""
    f = Function("QuantizeLinear", None, [int(narrow_range), _dtype_code(dtype)], [], round_mode,
                 args=dict(round_mode=round_mode, narrow_range=narrow_range, dtype=_dtype_code(dtype)))
    return f(x, scale, zero_point, outputs=outputs)


def dequantize_linear(x, scale, zero_point, n_outputs=-1, outputs=None):
    """``(x - zero_point) * scale`` (functions.yaml:7602-7640)."""
    f = Function("DequantizeLinear", None, [], [])
    return f(x, scale, zero_point, outputs=outputs)


def prune(x, rate=0.9, n_outputs=-1, outputs=None):
    """Zero the ``rate`` fraction of smallest magnitudes (functions.yaml:7521-7555)."""
    f = Function("Prune", None, [], [rate], args=dict(rate=rate))
    return f(x, outputs=outputs)


def sink(*x, **kw):
    """Joins graph outputs into one terminal variable of shape (); its backward seeds every input's gradient with
    ones when ``one_input_grad`` is set (functions.yaml, Sink; src/nbla/function/generic/sink.cpp:25-48)."""
    one_input_grad = bool(kw.pop("one_input_grad", True))
    outputs = kw.pop("outputs", None)
    kw.pop("n_outputs", None)
    if kw:
        raise TypeError("sink: unexpected arguments %r" % sorted(kw))
    f = Function("Sink", None, [int(one_input_grad)], args=dict(one_input_grad=one_input_grad))
    return f(*x, outputs=outputs)


def _dtype_code(dtype):
    """nbla::dtypes code of a numpy dtype (int8 -> 1, uint8 -> 2); integers pass through."""
    if isinstance(dtype, int):
        return dtype
    import numpy as np
    code = {np.dtype(np.int8): 1, np.dtype(np.uint8): 2}.get(np.dtype(dtype))
    if code is None:
        raise ValueError("quantize_linear: dtype must be int8 or uint8, not %r" % (dtype,))
    return code
