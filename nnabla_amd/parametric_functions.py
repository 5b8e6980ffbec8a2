"""``PF.*``: the parametric layers built on the quantization functions, with nnabla's names, argument order,
parameter names and scopes (python/src/nnabla/parametric_functions.py:125-181, 314-558, 559-637, 941-1186,
2290-2966, 2967-3400).  Every layer registers its parameters in the current parameter scope under the scope name
nnabla uses ("affine", "bicon_affine", "bwn_conv", "fp_quantized_affine", ...) and accepts ``name=`` to wrap that
scope in another one.

All layers share one skeleton -- create W (and b), derive the weights the product sees, call the product -- so they
are written as small "weight recipes" handed to ``_affine_layer`` / ``_conv_layer``.
"""
import functools

import numpy as np

from . import functions as F
from .initializer import ConstantInitializer, UniformInitializer, calc_uniform_lim_glorot
from .parameter import get_parameter_or_create, parameter_scope


def parametric_function_api(scope_name):
    """Runs the layer under ``parameter_scope(scope_name)``, itself under ``parameter_scope(name)`` when the added
    keyword ``name`` is given (parametric_functions.py:28-122)."""
    def wrap(func):
        @functools.wraps(func)
        def layer(*args, **kw):
            name = kw.pop("name", None)
            if name is None:
                with parameter_scope(scope_name):
                    return func(*args, **kw)
            with parameter_scope(name):
                with parameter_scope(scope_name):
                    return func(*args, **kw)
        layer.__scope_name__ = scope_name
        return layer
    return wrap


# ------------------------------------------------------------------------------------------------ skeletons

def _outmaps_list(n_outmaps):
    return list(n_outmaps) if hasattr(n_outmaps, '__iter__') else [n_outmaps]


def _affine_shapes(inp, n_outmaps, base_axis):
    outs = _outmaps_list(n_outmaps)
    inmaps = int(np.prod(inp.shape[base_axis:]))
    return inmaps, outs, int(np.prod(outs))


def _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng, with_bias=True):
    inmaps, outs, n_out = _affine_shapes(inp, n_outmaps, base_axis)
    if w_init is None:
        w_init = UniformInitializer(calc_uniform_lim_glorot(inmaps, n_out), rng=rng)
    if with_bias and b_init is None:
        b_init = ConstantInitializer()
    return [inmaps] + outs, outs, w_init, b_init


def _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng, with_bias=True):
    channels = inp.shape[base_axis]
    if w_init is None:
        w_init = UniformInitializer(calc_uniform_lim_glorot(channels, outmaps, tuple(kernel)), rng=rng)
    if with_bias and b_init is None:
        b_init = ConstantInitializer()
    return (outmaps, channels // group) + tuple(kernel), (outmaps,), w_init, b_init


def _float_pair(w_shape, b_shape, w_init, b_init, fix_parameters, with_bias):
    w = get_parameter_or_create("W", w_shape, w_init, True, not fix_parameters)
    b = get_parameter_or_create("b", b_shape, b_init, True, not fix_parameters) if with_bias else None
    return w, b


def _derived(param, name, init, enabled, derive):
    """The weights the product sees: ``derive(param, outputs=[<name>.data])`` written into a registered,
    non-trainable companion parameter, or the parameter itself when the derivation is switched off."""
    if param is None or not enabled:
        return param
    companion = get_parameter_or_create(name, param.shape, init, False)
    out = derive(param, outputs=[companion.data])
    out.persistent = True
    return out


# --------------------------------------------------------------------------------------------- plain layers

@parametric_function_api("affine")
def affine(inp, n_outmaps, base_axis=1, w_init=None, b_init=None, fix_parameters=False, rng=None, with_bias=True,
           apply_w=None, apply_b=None):
    w_shape, b_shape, w_init, b_init = _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng, with_bias)
    w, b = _float_pair(w_shape, b_shape, w_init, b_init, fix_parameters, with_bias)
    if apply_w is not None:
        w = apply_w(w)
    if b is not None and apply_b is not None:
        b = apply_b(b)
    return F.affine(inp, w, b, base_axis)


@parametric_function_api("conv")
def convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1, channel_last=False, w_init=None,
                b_init=None, base_axis=1, fix_parameters=False, rng=None, with_bias=True, apply_w=None,
                apply_b=None):
    if channel_last:
        raise NotImplementedError("channel_last convolutions are not implemented on this path.")
    w_shape, b_shape, w_init, b_init = _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng,
                                                   with_bias)
    w, b = _float_pair(w_shape, b_shape, w_init, b_init, fix_parameters, with_bias)
    if apply_w is not None:
        w = apply_w(w)
    if b is not None and apply_b is not None:
        b = apply_b(b)
    return F.convolution(inp, w, b, base_axis, pad, stride, dilation, group, channel_last)


# ------------------------------------------------------------------------------ binary and INQ layers

def _binary_params(w_shape, b_shape, w_init, wb_init, b_init, fix_parameters, with_bias, alpha_shape=None):
    w = get_parameter_or_create("W", w_shape, w_init, True, not fix_parameters)
    wb = get_parameter_or_create("Wb", w_shape, wb_init, False)
    alpha = None
    if alpha_shape is not None:
        alpha = get_parameter_or_create("alpha", alpha_shape, ConstantInitializer(0), False)
    b = get_parameter_or_create("b", b_shape, b_init, True, not fix_parameters) if with_bias else None
    return w, wb, alpha, b


@parametric_function_api("bicon_affine")
def binary_connect_affine(inp, n_outmaps, base_axis=1, quantize_zero_to=1.0, w_init=None, wb_init=None, b_init=None,
                          fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng)
    wb_init = wb_init if wb_init is not None else _affine_inits(inp, n_outmaps, base_axis, None, None, rng)[2]
    w, wb, _, b = _binary_params(w_shape, b_shape, w_init, wb_init, b_init, fix_parameters, with_bias)
    return F.binary_connect_affine(inp, w, wb, b, base_axis, quantize_zero_to)


@parametric_function_api("bwn_affine")
def binary_weight_affine(inp, n_outmaps, base_axis=1, quantize_zero_to=1.0, w_init=None, wb_init=None, b_init=None,
                         fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng)
    wb_init = wb_init if wb_init is not None else _affine_inits(inp, n_outmaps, base_axis, None, None, rng)[2]
    w, wb, alpha, b = _binary_params(w_shape, b_shape, w_init, wb_init, b_init, fix_parameters, with_bias, b_shape)
    return F.binary_weight_affine(inp, w, wb, alpha, b, base_axis, quantize_zero_to)


@parametric_function_api("bicon_conv")
def binary_connect_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1,
                               quantize_zero_to=1.0, w_init=None, wb_init=None, b_init=None, base_axis=1,
                               fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng)
    wb_init = wb_init if wb_init is not None else _conv_inits(inp, outmaps, kernel, group, base_axis, None, None,
                                                              rng)[2]
    w, wb, _, b = _binary_params(w_shape, b_shape, w_init, wb_init, b_init, fix_parameters, with_bias)
    return F.binary_connect_convolution(inp, w, wb, b, base_axis, pad, stride, dilation, group, quantize_zero_to)


@parametric_function_api("bwn_conv")
def binary_weight_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1,
                              quantize_zero_to=1.0, w_init=None, wb_init=None, b_init=None, base_axis=1,
                              fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng)
    wb_init = wb_init if wb_init is not None else _conv_inits(inp, outmaps, kernel, group, base_axis, None, None,
                                                              rng)[2]
    w, wb, alpha, b = _binary_params(w_shape, b_shape, w_init, wb_init, b_init, fix_parameters, with_bias, b_shape)
    return F.binary_weight_convolution(inp, w, wb, alpha, b, base_axis, pad, stride, dilation, group,
                                       quantize_zero_to)


def _inq_params(w_shape, b_shape, w_init, i_init, b_init, fix_parameters, with_bias):
    w = get_parameter_or_create("W", w_shape, w_init, True, not fix_parameters)
    i = get_parameter_or_create("I", w_shape, i_init if i_init is not None else ConstantInitializer(), False)
    if i._dtype(0) != np.dtype(np.int32):
        i.set_data(i.d, np.int32)  # the indicators are integers (the function's TI type)
    b = get_parameter_or_create("b", b_shape, b_init, True, not fix_parameters) if with_bias else None
    return w, i, b


@parametric_function_api("inq_affine")
def inq_affine(inp, n_outmaps, base_axis=1, num_bits=4, inq_iterations=(), selection_algorithm='random', seed=-1,
               w_init=None, i_init=None, b_init=None, fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng)
    w, i, b = _inq_params(w_shape, b_shape, w_init, i_init, b_init, fix_parameters, with_bias)
    return F.inq_affine(inp, w, i, b, base_axis, num_bits, inq_iterations, selection_algorithm, seed)


@parametric_function_api("inq_conv")
def inq_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1, num_bits=4,
                    inq_iterations=(), selection_algorithm='random', seed=-1, w_init=None, i_init=None, b_init=None,
                    base_axis=1, fix_parameters=False, rng=None, with_bias=True):
    w_shape, b_shape, w_init, b_init = _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng)
    w, i, b = _inq_params(w_shape, b_shape, w_init, i_init, b_init, fix_parameters, with_bias)
    return F.inq_convolution(inp, w, i, b, base_axis, pad, stride, dilation, group, num_bits, inq_iterations,
                             selection_algorithm, seed)


# -------------------------------------------------------- layers that quantize (or prune) W and b first

def _affine_layer(inp, n_outmaps, base_axis, w_init, b_init, fix_parameters, rng, with_bias, derive_w, derive_b):
    w_shape, b_shape, w_init, b_init = _affine_inits(inp, n_outmaps, base_axis, w_init, b_init, rng, with_bias)
    w, b = _float_pair(w_shape, b_shape, w_init, b_init, fix_parameters, with_bias)
    w_q = _derived(w, "W_q", w_init, derive_w is not None, derive_w)
    b_q = _derived(b, "b_q", b_init, derive_b is not None, derive_b)
    return F.affine(inp, w_q, b_q, base_axis)


def _conv_layer(inp, outmaps, kernel, pad, stride, dilation, group, channel_last, base_axis, w_init, b_init,
                fix_parameters, rng, with_bias, derive_w, derive_b):
    if channel_last:
        raise NotImplementedError("channel_last convolutions are not implemented on this path.")
    w_shape, b_shape, w_init, b_init = _conv_inits(inp, outmaps, kernel, group, base_axis, w_init, b_init, rng,
                                                   with_bias)
    w, b = _float_pair(w_shape, b_shape, w_init, b_init, fix_parameters, with_bias)
    w_q = _derived(w, "W_q", w_init, derive_w is not None, derive_w)
    b_q = _derived(b, "b_q", b_init, derive_b is not None, derive_b)
    return F.convolution(inp, w_q, b_q, base_axis, pad, stride, dilation, group, channel_last)


def _fp(quantize, sign, n, delta, ste):
    if not quantize:
        return None
    return lambda v, outputs: F.fixed_point_quantize(v, sign=sign, n=n, delta=delta, ste_fine_grained=ste,
                                                     outputs=outputs)


def _pow2(quantize, sign, with_zero, n, m, ste):
    if not quantize:
        return None
    return lambda v, outputs: F.pow2_quantize(v, sign=sign, with_zero=with_zero, n=n, m=m, ste_fine_grained=ste,
                                              outputs=outputs)


def _pruner(prune, rate):
    if not prune:
        return None
    return lambda v, outputs: F.prune(v, rate, outputs=outputs)


@parametric_function_api("fp_quantized_affine")
def fixed_point_quantized_affine(inp, n_outmaps, base_axis=1, w_init=None, b_init=None, fix_parameters=False,
                                 rng=None, with_bias=True, quantize_w=True, sign_w=True, n_w=8, delta_w=2 ** -4,
                                 ste_fine_grained_w=True, quantize_b=True, sign_b=True, n_b=8, delta_b=2 ** -4,
                                 ste_fine_grained_b=True):
    return _affine_layer(inp, n_outmaps, base_axis, w_init, b_init, fix_parameters, rng, with_bias,
                         _fp(quantize_w, sign_w, n_w, delta_w, ste_fine_grained_w),
                         _fp(quantize_b, sign_b, n_b, delta_b, ste_fine_grained_b))


@parametric_function_api("fp_quantized_conv")
def fixed_point_quantized_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1,
                                      channel_last=False, w_init=None, b_init=None, base_axis=1,
                                      fix_parameters=False, rng=None, with_bias=True, quantize_w=True, sign_w=True,
                                      n_w=8, delta_w=2 ** -4, ste_fine_grained_w=True, quantize_b=True, sign_b=True,
                                      n_b=8, delta_b=2 ** -4, ste_fine_grained_b=True):
    return _conv_layer(inp, outmaps, kernel, pad, stride, dilation, group, channel_last, base_axis, w_init, b_init,
                       fix_parameters, rng, with_bias, _fp(quantize_w, sign_w, n_w, delta_w, ste_fine_grained_w),
                       _fp(quantize_b, sign_b, n_b, delta_b, ste_fine_grained_b))


@parametric_function_api("pow2_quantized_affine")
def pow2_quantized_affine(inp, n_outmaps, base_axis=1, w_init=None, b_init=None, fix_parameters=False, rng=None,
                          with_bias=True, quantize_w=True, sign_w=True, with_zero_w=False, n_w=8, m_w=2,
                          ste_fine_grained_w=True, quantize_b=True, sign_b=True, with_zero_b=False, n_b=8, m_b=2,
                          ste_fine_grained_b=True):
    return _affine_layer(inp, n_outmaps, base_axis, w_init, b_init, fix_parameters, rng, with_bias,
                         _pow2(quantize_w, sign_w, with_zero_w, n_w, m_w, ste_fine_grained_w),
                         _pow2(quantize_b, sign_b, with_zero_b, n_b, m_b, ste_fine_grained_b))


@parametric_function_api("pow2_quantized_conv")
def pow2_quantized_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1, w_init=None,
                               b_init=None, base_axis=1, fix_parameters=False, rng=None, with_bias=True,
                               quantize_w=True, with_zero_w=False, sign_w=True, n_w=8, m_w=2,
                               ste_fine_grained_w=True, quantize_b=True, with_zero_b=False, sign_b=True, n_b=8,
                               m_b=2, ste_fine_grained_b=True):
    return _conv_layer(inp, outmaps, kernel, pad, stride, dilation, group, False, base_axis, w_init, b_init,
                       fix_parameters, rng, with_bias,
                       _pow2(quantize_w, sign_w, with_zero_w, n_w, m_w, ste_fine_grained_w),
                       _pow2(quantize_b, sign_b, with_zero_b, n_b, m_b, ste_fine_grained_b))


@parametric_function_api("pruned_affine")
def pruned_affine(inp, n_outmaps, base_axis=1, w_init=None, b_init=None, fix_parameters=False, rng=None,
                  with_bias=True, prune_w=True, rate_w=0.9, prune_b=True, rate_b=0.9):
    return _affine_layer(inp, n_outmaps, base_axis, w_init, b_init, fix_parameters, rng, with_bias,
                         _pruner(prune_w, rate_w), _pruner(prune_b, rate_b))


@parametric_function_api("pruned_conv")
def pruned_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1, channel_last=False,
                       w_init=None, b_init=None, base_axis=1, fix_parameters=False, rng=None, with_bias=True,
                       prune_w=True, rate_w=0.9, prune_b=True, rate_b=0.9):
    return _conv_layer(inp, outmaps, kernel, pad, stride, dilation, group, channel_last, base_axis, w_init, b_init,
                       fix_parameters, rng, with_bias, _pruner(prune_w, rate_w), _pruner(prune_b, rate_b))


# --------------------------------------------------------------------------------------- min-max quantization

@parametric_function_api("min_max_quantize")
def min_max_quantize(x, ql_min=0, ql_max=255, decay=0.999, x_min_max=False, ema=False, ste_fine_grained=True,
                     eps=0.01, qr_min_init=None, qr_max_init=None, fix_parameters=False, outputs=None):
    """Min-max quantization with its ranges kept as parameters ``qr_min`` / ``qr_max`` (and ``ql_min`` / ``ql_max``
    when given as numbers), shaped ``[1] * x.ndim`` (parametric_functions.py:2971-3098)."""
    ones = [1] * x.ndim
    if isinstance(ql_min, (int, float)):
        ql_min = get_parameter_or_create("ql_min", ones, np.full(ones, ql_min, np.float32), False, False)
    if isinstance(ql_max, (int, float)):
        ql_max = get_parameter_or_create("ql_max", ones, np.full(ones, ql_max, np.float32), False, False)
    qr_min_init = qr_min_init if qr_min_init else ConstantInitializer(-6.0)
    qr_max_init = qr_max_init if qr_max_init else ConstantInitializer(6.0)
    learnable = not (x_min_max and ema)
    qr_min = get_parameter_or_create("qr_min", ql_min.shape, qr_min_init, learnable, not fix_parameters)
    qr_max = get_parameter_or_create("qr_max", ql_min.shape, qr_max_init, learnable, not fix_parameters)
    return F.min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, decay, x_min_max, ema, ste_fine_grained, eps,
                              outputs=outputs)


def _min_max(quantize, ql_min, ql_max, use_min_max, qr_min_init, qr_max_init, default_range, ste, eps, fix_parameters,
             scope):
    if not quantize:
        return None
    qr_min_init = qr_min_init if qr_min_init is not None else ConstantInitializer(-default_range)
    qr_max_init = qr_max_init if qr_max_init is not None else ConstantInitializer(default_range)
    return lambda v, outputs: min_max_quantize(v, ql_min, ql_max, 0.999, use_min_max, False, ste, eps, qr_min_init,
                                               qr_max_init, fix_parameters, outputs=outputs, name=scope)


@parametric_function_api("min_max_quantized_affine")
def min_max_quantized_affine(inp, n_outmaps, base_axis=1, w_init=None, b_init=None, fix_parameters=False, rng=None,
                             with_bias=True, quantize_w=True, ql_min_w=0, ql_max_w=255, w_min_max=False,
                             qr_min_w_init=None, qr_max_w_init=None, ste_fine_grained_w=True, quantize_b=True,
                             ql_min_b=0, ql_max_b=255, b_min_max=False, qr_min_b_init=None, qr_max_b_init=None,
                             ste_fine_grained_b=True, eps=0.01):
    return _affine_layer(
        inp, n_outmaps, base_axis, w_init, b_init, fix_parameters, rng, with_bias,
        _min_max(quantize_w, ql_min_w, ql_max_w, w_min_max, qr_min_w_init, qr_max_w_init, 2.0, ste_fine_grained_w, eps,
                 fix_parameters, "min_max_quantize_w"),
        _min_max(quantize_b, ql_min_b, ql_max_b, b_min_max, qr_min_b_init, qr_max_b_init, 6.0, ste_fine_grained_b, eps,
                 fix_parameters, "min_max_quantize_b"))


@parametric_function_api("min_max_quantized_conv")
def min_max_quantized_convolution(inp, outmaps, kernel, pad=None, stride=None, dilation=None, group=1,
                                  channel_last=False, w_init=None, b_init=None, base_axis=1, fix_parameters=False,
                                  rng=None, with_bias=True, quantize_w=True, ql_min_w=0, ql_max_w=255,
                                  w_min_max=False, qr_min_w_init=None, qr_max_w_init=None, ste_fine_grained_w=True,
                                  quantize_b=True, ql_min_b=0, ql_max_b=255, b_min_max=False, qr_min_b_init=None,
                                  qr_max_b_init=None, ste_fine_grained_b=True, eps=0.01):
    return _conv_layer(
        inp, outmaps, kernel, pad, stride, dilation, group, channel_last, base_axis, w_init, b_init, fix_parameters,
        rng, with_bias,
        _min_max(quantize_w, ql_min_w, ql_max_w, w_min_max, qr_min_w_init, qr_max_w_init, 2.0, ste_fine_grained_w, eps,
                 fix_parameters, "min_max_quantize_w"),
        _min_max(quantize_b, ql_min_b, ql_max_b, b_min_max, qr_min_b_init, qr_max_b_init, 6.0, ste_fine_grained_b, eps,
                 fix_parameters, "min_max_quantize_b"))
