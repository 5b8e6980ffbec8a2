"""ctypes front-end of the CPU oracle (``libnbla_quant_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the CPU-baseline leg of ``bench.py``.  The product package never imports
this module.  Every function takes and returns numpy arrays (fp32 / int32,
C-contiguous) and maps one-to-one onto an ``orc_*`` entry point, which in turn
cites the nnabla file:line it restates; ``range_recorder`` and ``recorder_scale``
(scalar bookkeeping of quantization-aware training) are numpy restatements
written here.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnbla_quant_oracle.so")

_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_int_p = ctypes.POINTER(ctypes.c_int)
_c_long_p = ctypes.POINTER(ctypes.c_long)


def build(force=False):
    """Compile the oracle with its Makefile (g++ -O3, no -march, no FMA)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_inq_create.restype = ctypes.c_void_p
        _lib.orc_bernoulli_create.restype = ctypes.c_void_p
        _lib.orc_inq_counter.restype = ctypes.c_long
    return _lib


class OracleError(ValueError):
    pass


def _check(rc, what):
    if rc != 0:
        raise OracleError("%s failed with nbla error code %d" % (what, rc))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_c_float_p)


def _ip(a):
    return a.ctypes.data_as(_c_int_p)


def _longs(seq):
    arr = (ctypes.c_long * len(seq))(*[int(v) for v in seq])
    return arr


def fixed_point_quantize(x, sign=True, n=8, delta=2.0 ** -4):
    x = _f32(x)
    y = np.empty_like(x)
    _check(lib().orc_fixed_point_quantize(_fp(x), _fp(y), ctypes.c_long(x.size), int(sign), int(n),
                                          ctypes.c_float(delta)), "fixed_point_quantize")
    return y


def pow2_quantize(x, sign=True, with_zero=True, n=8, m=1):
    x = _f32(x)
    y = np.empty_like(x)
    _check(lib().orc_pow2_quantize(_fp(x), _fp(y), ctypes.c_long(x.size), int(sign), int(with_zero), int(n),
                                   int(m)), "pow2_quantize")
    return y


def round_log2(a):
    return lib().orc_round_log2(ctypes.c_float(a))


def inq_exponent(a):
    return lib().orc_inq_exponent(ctypes.c_float(a))


def inq_n1(a):
    return lib().orc_inq_n1(ctypes.c_float(a))


def min_max_reduce(x, qshape):
    x = _f32(x)
    qshape = tuple(int(s) for s in qshape)
    mn = np.empty(qshape, np.float32)
    mx = np.empty(qshape, np.float32)
    lib().orc_min_max_reduce(_fp(x), _longs(x.shape), x.ndim, _longs(qshape), _fp(mn), _fp(mx))
    return mn, mx


def min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, decay=0.999, x_min_max=False, ema=False, eps=0.01):
    """Returns (y, qr_min_new, qr_max_new, scale); the inputs are not modified."""
    x = _f32(x)
    qr_min = _f32(qr_min).copy()
    qr_max = _f32(qr_max).copy()
    ql_min = _f32(ql_min)
    ql_max = _f32(ql_max)
    assert qr_min.shape == qr_max.shape == ql_min.shape == ql_max.shape and qr_min.ndim == x.ndim
    y = np.empty_like(x)
    scale = np.empty_like(qr_min)
    _check(lib().orc_min_max_quantize(_fp(x), _fp(y), _longs(x.shape), x.ndim, _longs(qr_min.shape), _fp(qr_min),
                                      _fp(qr_max), _fp(ql_min), _fp(ql_max), ctypes.c_float(decay), int(x_min_max),
                                      int(ema), ctypes.c_float(eps), _fp(scale)), "min_max_quantize")
    return y, qr_min, qr_max, scale


def _opt(a, want, like_shape):
    if not want:
        return None
    return np.zeros(like_shape, np.float32) if a is None else _f32(a).copy()


def affine_backward(dy, x, W, dx=None, dW=None, db=None, want=(True, True, True)):
    """(dx, dW, db) of y = x.W + b (affine.cpp:98-140); gradients passed in are accumulated onto."""
    dy, x, W = _f32(dy), _f32(x), _f32(W)
    M, K = x.shape
    N = W.size // K
    odx, odw, odb = _opt(dx, want[0], (M, K)), _opt(dW, want[1], W.shape), _opt(db, want[2], (N,))
    nul = ctypes.POINTER(ctypes.c_float)()
    _check(lib().orc_affine_backward(_fp(dy), _fp(x), _fp(W), _fp(odx) if want[0] else nul,
                                     _fp(odw) if want[1] else nul, _fp(odb) if want[2] else nul, ctypes.c_long(M),
                                     ctypes.c_long(K), ctypes.c_long(N), int(dx is not None), int(dW is not None),
                                     int(db is not None)), "affine_backward")
    return odx, odw, odb


def binary_affine_backward(dy, x, W, alpha=None, quantize_zero_to=1.0, dx=None, dW=None, db=None,
                           want=(True, True, True)):
    """Backward of BinaryWeightAffine (alpha given) / BinaryConnectAffine (alpha None)."""
    dy, x, W = _f32(dy), _f32(x), _f32(W)
    M, K = x.shape
    N = W.size // K
    odx, odw, odb = _opt(dx, want[0], (M, K)), _opt(dW, want[1], W.shape), _opt(db, want[2], (N,))
    nul = ctypes.POINTER(ctypes.c_float)()
    al = _f32(alpha) if alpha is not None else None
    _check(lib().orc_binary_affine_backward(_fp(dy), _fp(x), _fp(W), _fp(al) if al is not None else nul,
                                            _fp(odx) if want[0] else nul, _fp(odw) if want[1] else nul,
                                            _fp(odb) if want[2] else nul, ctypes.c_long(M), ctypes.c_long(K),
                                            ctypes.c_long(N), ctypes.c_float(quantize_zero_to), int(dx is not None),
                                            int(dW is not None), int(db is not None)), "binary_affine_backward")
    return odx, odw, odb


def fixed_point_quantize_backward(dy, x, sign=True, n=8, delta=2.0 ** -4, ste_fine_grained=True, dx=None):
    """dx (accumulated onto the given dx when one is passed), fixed_point_quantize.cpp:69-127."""
    dy, x = _f32(dy), _f32(x)
    out = np.zeros_like(x) if dx is None else _f32(dx).copy()
    _check(lib().orc_fixed_point_quantize_backward(_fp(dy), _fp(x), _fp(out), ctypes.c_long(x.size), int(sign), int(n),
                                                   ctypes.c_float(delta), int(ste_fine_grained), int(dx is not None)),
           "fixed_point_quantize_backward")
    return out


def pow2_quantize_backward(dy, x, sign=True, with_zero=True, n=8, m=1, ste_fine_grained=True, dx=None):
    dy, x = _f32(dy), _f32(x)
    out = np.zeros_like(x) if dx is None else _f32(dx).copy()
    _check(lib().orc_pow2_quantize_backward(_fp(dy), _fp(x), _fp(out), ctypes.c_long(x.size), int(sign),
                                            int(with_zero), int(n), int(m), int(ste_fine_grained),
                                            int(dx is not None)), "pow2_quantize_backward")
    return out


def min_max_quantize_backward(dy, x, qr_min, qr_max, ql_min, ql_max, scale, ste_fine_grained=True, x_min_max=False,
                              ema=False, dx=None, g_qr_min=None, g_qr_max=None, want_x=True, want_min=True,
                              want_max=True):
    """Returns (dx, g_qr_min, g_qr_max); a gradient passed in is accumulated onto, min_max_quantize.cpp:225-350."""
    dy, x = _f32(dy), _f32(x)
    qs = [_f32(q) for q in (qr_min, qr_max, ql_min, ql_max, scale)]
    odx = (np.zeros_like(x) if dx is None else _f32(dx).copy()) if want_x else None
    omin = (np.zeros_like(qs[0]) if g_qr_min is None else _f32(g_qr_min).copy()) if want_min else None
    omax = (np.zeros_like(qs[0]) if g_qr_max is None else _f32(g_qr_max).copy()) if want_max else None
    nul = ctypes.POINTER(ctypes.c_float)()
    _check(lib().orc_min_max_quantize_backward(
        _fp(dy), _fp(x), _fp(odx) if want_x else nul, _longs(x.shape), x.ndim, _longs(qs[0].shape), _fp(qs[0]),
        _fp(qs[1]), _fp(qs[2]), _fp(qs[3]), _fp(qs[4]), _fp(omin) if want_min else nul,
        _fp(omax) if want_max else nul, int(ste_fine_grained), int(x_min_max), int(ema), int(dx is not None),
        int(g_qr_min is not None), int(g_qr_max is not None)), "min_max_quantize_backward")
    return odx, omin, omax


def sign(x, alpha0=1.0):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_sign(_fp(x), _fp(y), ctypes.c_long(x.size), ctypes.c_float(alpha0))
    return y


def affine(x, w, b=None):
    x = _f32(x)
    w = _f32(w)
    M, K = x.shape
    N = w.size // K
    b = None if b is None else _f32(b)
    y = np.empty((M, N), np.float32)
    _check(lib().orc_affine(_fp(x), _fp(w), _fp(b), _fp(y), ctypes.c_long(M), ctypes.c_long(K), ctypes.c_long(N)),
           "affine")
    return y


def binary_weight_prepare(W, quantize_zero_to=1.0, want_scaled=False):
    """Returns (Wb, alpha[, scaled]) for W viewed as [K, N]."""
    W = _f32(W)
    K = W.shape[0]
    N = W.size // K
    Wb = np.empty_like(W)
    alpha = np.empty(N, np.float32)
    scaled = np.empty_like(W) if want_scaled else None
    lib().orc_binary_weight_prepare(_fp(W), _fp(Wb), _fp(alpha), _fp(scaled), ctypes.c_long(K), ctypes.c_long(N),
                                    ctypes.c_float(quantize_zero_to))
    return (Wb, alpha, scaled) if want_scaled else (Wb, alpha)


def binary_weight_affine(x, W, b=None, quantize_zero_to=1.0):
    """Returns (y, Wb, alpha)."""
    x = _f32(x)
    W = _f32(W)
    M, K = x.shape
    N = W.size // K
    b = None if b is None else _f32(b)
    Wb = np.empty_like(W)
    alpha = np.empty(N, np.float32)
    y = np.empty((M, N), np.float32)
    _check(lib().orc_binary_weight_affine(_fp(x), _fp(W), _fp(Wb), _fp(alpha), _fp(b), _fp(y), ctypes.c_long(M),
                                          ctypes.c_long(K), ctypes.c_long(N), ctypes.c_float(quantize_zero_to)),
           "binary_weight_affine")
    return y, Wb, alpha


def binary_connect_affine(x, W, b=None, quantize_zero_to=1.0):
    """Returns (y, Wb)."""
    x = _f32(x)
    W = _f32(W)
    M, K = x.shape
    N = W.size // K
    b = None if b is None else _f32(b)
    Wb = np.empty_like(W)
    y = np.empty((M, N), np.float32)
    _check(lib().orc_binary_connect_affine(_fp(x), _fp(W), _fp(Wb), _fp(b), _fp(y), ctypes.c_long(M),
                                           ctypes.c_long(K), ctypes.c_long(N), ctypes.c_float(quantize_zero_to)),
           "binary_connect_affine")
    return y, Wb


def _conv_args(x, W, pad, stride, dilation, group):
    x = _f32(x)
    W = _f32(W)
    nd = W.ndim - 2
    outer = int(np.prod(x.shape[:x.ndim - nd - 1], dtype=np.int64))
    C = x.shape[x.ndim - nd - 1]
    in_sp = x.shape[x.ndim - nd:]
    O = W.shape[0]
    kernel = W.shape[2:]
    pad = tuple(pad) if pad is not None else (0,) * nd
    stride = tuple(stride) if stride is not None else (1,) * nd
    dilation = tuple(dilation) if dilation is not None else (1,) * nd
    out_sp = (ctypes.c_long * nd)()
    tail = (ctypes.c_long(outer), ctypes.c_long(C), nd, _longs(in_sp), ctypes.c_long(O), _longs(kernel), _longs(pad),
            _longs(stride), _longs(dilation), ctypes.c_long(group))
    _check(lib().orc_convolution(None, None, None, None, *tail, out_sp), "convolution geometry")
    yshape = tuple(x.shape[:x.ndim - nd - 1]) + (O,) + tuple(out_sp)
    return x, W, tail, yshape


def convolution(x, W, b=None, pad=None, stride=None, dilation=None, group=1):
    x, W, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
    b = None if b is None else _f32(b)
    y = np.empty(yshape, np.float32)
    _check(lib().orc_convolution(_fp(x), _fp(W), _fp(b), _fp(y), *tail, None), "convolution")
    return y


def binary_weight_convolution(x, W, b=None, pad=None, stride=None, dilation=None, group=1, quantize_zero_to=1.0):
    """Returns (y, Wb, alpha)."""
    x, W, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
    b = None if b is None else _f32(b)
    y = np.empty(yshape, np.float32)
    Wb = np.empty_like(W)
    alpha = np.empty(W.shape[0], np.float32)
    _check(lib().orc_binary_weight_convolution(_fp(x), _fp(W), _fp(Wb), _fp(alpha), _fp(b), _fp(y), *tail,
                                               ctypes.c_float(quantize_zero_to)), "binary_weight_convolution")
    return y, Wb, alpha


def binary_connect_convolution(x, W, b=None, pad=None, stride=None, dilation=None, group=1, quantize_zero_to=1.0):
    """Returns (y, Wb)."""
    x, W, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
    b = None if b is None else _f32(b)
    y = np.empty(yshape, np.float32)
    Wb = np.empty_like(W)
    _check(lib().orc_binary_connect_convolution(_fp(x), _fp(W), _fp(Wb), _fp(b), _fp(y), *tail,
                                                ctypes.c_float(quantize_zero_to)), "binary_connect_convolution")
    return y, Wb


def convolution_backward(dy, x, W, pad=None, stride=None, dilation=None, group=1, dx=None, dW=None, db=None,
                         want=(True, True, True)):
    """(dx, dW, db) of Convolution (convolution.cpp:199-283); gradients passed in are accumulated onto."""
    x, W, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
    dy = _f32(dy).reshape(yshape)
    odx, odw, odb = _opt(dx, want[0], x.shape), _opt(dW, want[1], W.shape), _opt(db, want[2], (W.shape[0],))
    nul = ctypes.POINTER(ctypes.c_float)()
    _check(lib().orc_convolution_backward(_fp(dy), _fp(x), _fp(W), _fp(odx) if want[0] else nul,
                                          _fp(odw) if want[1] else nul, _fp(odb) if want[2] else nul, *tail,
                                          int(dx is not None), int(dW is not None), int(db is not None)),
           "convolution_backward")
    return odx, odw, odb


def binary_convolution_backward(dy, x, W, alpha=None, pad=None, stride=None, dilation=None, group=1,
                                quantize_zero_to=1.0, dx=None, dW=None, db=None, want=(True, True, True)):
    """Backward of BinaryWeightConvolution (alpha given) / BinaryConnectConvolution (alpha None)."""
    x, W, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
    dy = _f32(dy).reshape(yshape)
    odx, odw, odb = _opt(dx, want[0], x.shape), _opt(dW, want[1], W.shape), _opt(db, want[2], (W.shape[0],))
    nul = ctypes.POINTER(ctypes.c_float)()
    al = _f32(alpha) if alpha is not None else None
    _check(lib().orc_binary_convolution_backward(_fp(dy), _fp(x), _fp(W), _fp(al) if al is not None else nul,
                                                 _fp(odx) if want[0] else nul, _fp(odw) if want[1] else nul,
                                                 _fp(odb) if want[2] else nul, *tail,
                                                 ctypes.c_float(quantize_zero_to), int(dx is not None),
                                                 int(dW is not None), int(db is not None)),
           "binary_convolution_backward")
    return odx, odw, odb


def _bshapes(x, scale, zero_point):
    x, scale, zero_point = _f32(x), _f32(scale), _f32(zero_point)
    assert x.ndim == scale.ndim == zero_point.ndim
    return x, scale, zero_point


def quantize_linear(x, scale, zero_point, round_mode="HALF_AWAY_FROM_ZERO", narrow_range=False, dtype=1):
    """Returns (y, zero_point after its in-place rounding); quantize_linear.cpp:97-117."""
    x, scale, zero_point = _bshapes(x, scale, zero_point)
    zp = zero_point.copy()
    y = np.empty_like(x)
    _check(lib().orc_quantize_linear(_fp(x), _fp(scale), _fp(zp), _fp(y), _longs(x.shape), _longs(scale.shape),
                                     _longs(zp.shape), x.ndim, int(round_mode == "HALF_TO_EVEN"), int(narrow_range),
                                     int(dtype)), "quantize_linear")
    return y, zp


def dequantize_linear(x, scale, zero_point):
    x, scale, zero_point = _bshapes(x, scale, zero_point)
    y = np.empty_like(x)
    _check(lib().orc_dequantize_linear(_fp(x), _fp(scale), _fp(zero_point), _fp(y), _longs(x.shape),
                                       _longs(scale.shape), _longs(zero_point.shape), x.ndim), "dequantize_linear")
    return y


def linear_quantize_backward(dy, scale, dequantize=False, dx=None):
    """dx (+)= dy / scale (QuantizeLinear) or dy * scale (DequantizeLinear)."""
    dy, scale = _f32(dy), _f32(scale)
    out = np.zeros_like(dy) if dx is None else _f32(dx).copy()
    _check(lib().orc_linear_quantize_backward(_fp(dy), _fp(scale), _fp(out), _longs(dy.shape), _longs(scale.shape),
                                              dy.ndim, int(dequantize), int(dx is not None)),
           "linear_quantize_backward")
    return out


def prune(x, rate=0.9):
    x = _f32(x)
    y = np.empty_like(x)
    _check(lib().orc_prune(_fp(x), _fp(y), ctypes.c_long(x.size), ctypes.c_float(rate)), "prune")
    return y


RECORDERS = ("MinMaxMinMaxRecorder", "AbsMaxRecorder", "MinMaxMvaRecorder", "MaxMaxRecorder", "MaxMvaRecorder")


def range_recorder(x, m, M, kind, decay=0.99):
    """One training-mode forward of a QAT range recorder: returns (m_new, M_new) as fp32 scalars (m_new is m unchanged
    for the one-sided kinds).  numpy restatement (no ``orc_*`` entry point) of python/src/nnabla/utils/qnn.py
    forward_impl :73-84 (MinMaxMinMax), :178-188 (AbsMax), :289-300 (MinMaxMva), :411-420 (MaxMax), :509-518
    (MaxMva), with Min / Max as ``min_max_reduce``, Minimum2 / Maximum2 as include/nbla/function/minimum2.hpp:41 /
    maximum2.hpp:41, and ``decay * m + (1 - decay) * mb`` as MulScalar, MulScalar, Add2 in fp32."""
    assert kind in RECORDERS
    f = np.float32
    x = _f32(x)
    src = np.abs(x) if kind == "AbsMaxRecorder" else x
    mb, Mb = min_max_reduce(src, (1,) * x.ndim)
    mb, Mb = f(mb.reshape(-1)[0]), f(Mb.reshape(-1)[0])
    m = None if m is None else f(np.asarray(m, np.float32).reshape(-1)[0])
    M = f(np.asarray(M, np.float32).reshape(-1)[0])
    if kind == "MinMaxMinMaxRecorder":
        return (m if m < mb else mb), (M if M > Mb else Mb)
    if kind in ("AbsMaxRecorder", "MaxMaxRecorder"):
        return m, (M if M > Mb else Mb)
    d, e = f(decay), f(1.0 - decay)
    if kind == "MinMaxMvaRecorder":
        return f(f(d * m) + f(e * mb)), f(f(d * M) + f(e * Mb))
    return m, f(f(d * M) + f(e * Mb))


def recorder_scale(m, M, kind, narrow_range=False, round_method="NOTROUND"):
    """QuantizeLinear scale from recorded statistics: qnn.py:126-139 for the two-sided recorders ((M - m) / levels,
    floored at 1e-24), :229-240 / :460-469 / :543-552 for the one-sided ones (2 M / levels); levels = 255, or 254
    with ``narrow_range``; then optionally moved to a power of two with the exponent rounded as asked."""
    levels = 254 if narrow_range else 255
    M = np.asarray(M, np.float32)
    if kind in ("MinMaxMinMaxRecorder", "MinMaxMvaRecorder"):
        scale = np.maximum(M - np.asarray(m, np.float32), np.float32(1e-24)) / np.float32(levels)
    else:
        scale = (np.float32(2) * M) / np.float32(levels)
    rnd = {"CEIL": np.ceil, "ROUND": np.round, "FLOOR": np.floor, "NOTROUND": None}[round_method]
    if rnd is not None:
        scale = np.float32(2) ** rnd(np.log(scale) / np.log(2))
    return np.asarray(scale, np.float32)


TRANSFORM_BINARY_OPS = ("sub2", "mul2", "div2", "add2", "pow2")   # the kernel library's operation codes 0..4


def _transform_binary_strides(shape0, shape1):
    """Output shape, merged axis groups and strides (0 along a broadcast group) of a two-input element-wise function:
    include/nbla/function/utils/base_transform_binary.hpp:58-205, statement by statement (the padding to three groups,
    :163-169, adds groups of size one and changes no index)."""
    s0, s1 = [int(v) for v in shape0], [int(v) for v in shape1]
    if len(s0) != len(s1):
        raise OracleError("Dimensions of inputs must match.")
    ndim = len(s0)
    oshape = []
    for i in range(ndim):
        if s0[i] != s1[i] and min(s0[i], s1[i]) != 1:
            raise OracleError("Broadcast dimension must be one.")
        oshape.append(max(s0[i], s1[i]))
    c0, c1, cy = [], [], []
    t0 = t1 = ty = 1
    for i in range(ndim - 1):
        t0, t1, ty = t0 * s0[i], t1 * s1[i], ty * oshape[i]
        kinds = [(s0[a] == s1[a], s0[a] == 1 and s1[a] != 1, s0[a] != 1 and s1[a] == 1) for a in (i, i + 1)]
        if not any(kinds[0][k] and kinds[1][k] for k in range(3)):
            c0.append(t0), c1.append(t1), cy.append(ty)
            t0 = t1 = ty = 1
    if ndim > 0:
        c0.append(t0 * s0[-1]), c1.append(t1 * s1[-1]), cy.append(ty * oshape[-1])
    while len(cy) < 3:
        c0.insert(0, 1), c1.insert(0, 1), cy.insert(0, 1)
    n = len(cy)
    st0, st1, sty = [1] * n, [1] * n, [1] * n
    for i in range(n - 2, -1, -1):
        st0[i], st1[i], sty[i] = st0[i + 1] * c0[i + 1], st1[i + 1] * c1[i + 1], sty[i + 1] * cy[i + 1]
    st0 = [st0[i] if c0[i] == cy[i] else 0 for i in range(n)]
    st1 = [st1[i] if c1[i] == cy[i] else 0 for i in range(n)]
    return tuple(oshape), cy, sty, st0, st1


def _transform_binary_indices(shape0, shape1):
    oshape, cy, sty, st0, st1 = _transform_binary_strides(shape0, shape1)
    size = int(np.prod(oshape, dtype=np.int64)) if len(oshape) else 1
    idx = np.arange(size, dtype=np.int64)
    idx0, idx1 = np.zeros(size, np.int64), np.zeros(size, np.int64)
    for i in range(len(cy)):                      # :270-277
        dim_idx = (idx // sty[i]) % cy[i]
        idx0 += dim_idx * st0[i]
        idx1 += dim_idx * st1[i]
    return oshape, idx0, idx1


def _binary_forward(op, a, b):
    f = np.float32
    with np.errstate(all="ignore"):
        if op == "sub2":
            return (a - b).astype(f)
        if op == "mul2":
            return (a * b).astype(f)
        if op == "div2":
            return (a / b).astype(f)
        if op == "add2":
            return (a + b).astype(f)
        return np.power(a, b).astype(f)           # std::pow on floats; numpy's powf, not bit-pinned


def _binary_grad(op, i, dy, a, b):
    """sub2.hpp:41, mul2.hpp:42, div2.hpp:44, bc_add2.hpp, pow2.hpp:44-47, every operation in fp32."""
    f = np.float32
    with np.errstate(all="ignore"):
        if op == "sub2":
            return dy if i == 0 else -dy
        if op == "mul2":
            return (dy * b).astype(f) if i == 0 else (dy * a).astype(f)
        if op == "div2":
            return (dy / b).astype(f) if i == 0 else ((-dy * a).astype(f) / (b * b).astype(f)).astype(f)
        if op == "add2":
            return dy
        if i == 0:
            return ((dy * b).astype(f) * np.power(a, (b - f(1)).astype(f)).astype(f)).astype(f)
        return ((dy * np.log(a).astype(f)).astype(f) * np.power(a, b).astype(f)).astype(f)


def transform_binary(op, x0, x1):
    """y = op(x0, x1) with broadcasting: transform_binary, utils/base_transform_binary.hpp:265-284 (every output index
    decomposed over the merged groups, operand indices through strides that are 0 along a broadcast group)."""
    assert op in TRANSFORM_BINARY_OPS
    oshape, idx0, idx1 = _transform_binary_indices(np.shape(x0), np.shape(x1))
    x0, x1 = _f32(x0), _f32(x1)
    return _binary_forward(op, x0.reshape(-1)[idx0], x1.reshape(-1)[idx1]).reshape(oshape)


def transform_binary_backward(op, i, dy, x0, x1, g=None):
    """Gradient of input i: transform_binary_grad0 / grad1, utils/base_transform_binary.hpp:286-336, on a gradient
    array that is zeroed first (:377-379 / :385-387) unless ``g`` (accumulation) is given: the terms are added one
    after the other in ascending output index, in fp32."""
    assert op in TRANSFORM_BINARY_OPS and i in (0, 1)
    shape0, shape1 = np.shape(x0), np.shape(x1)
    oshape, idx0, idx1 = _transform_binary_indices(shape0, shape1)
    assert tuple(np.shape(dy)) == tuple(oshape)
    dy, x0, x1 = _f32(dy), _f32(x0), _f32(x1)
    terms = _binary_grad(op, i, dy.reshape(-1), x0.reshape(-1)[idx0], x1.reshape(-1)[idx1])
    shape = shape0 if i == 0 else shape1
    out = np.zeros(shape, np.float32) if g is None else _f32(g).copy().reshape(shape)
    np.add.at(out.reshape(-1), idx0 if i == 0 else idx1, terms)      # unbuffered: in index order, in fp32
    return out


class Inq(object):
    """Stateful INQ weight logic (one object per INQAffine / INQConvolution)."""

    def __init__(self, size, num_bits=4, inq_iterations=(), selection_algorithm="largest_abs", seed=-1):
        its = (ctypes.c_int * max(1, len(inq_iterations)))(*[int(i) for i in inq_iterations])
        self._h = lib().orc_inq_create(ctypes.c_long(size), int(num_bits), its, len(inq_iterations),
                                       selection_algorithm.encode(), int(seed))
        if not self._h:
            raise OracleError("invalid selection algorithm %r" % (selection_algorithm,))
        self._h = ctypes.c_void_p(self._h)
        self.size = size

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_inq_destroy(self._h)
            self._h = None

    @property
    def counter(self):
        return lib().orc_inq_counter(self._h)

    def quantize_weights(self, W, I):
        """Steps A-C in place on fp32 W and int32 I; returns (n1, n2)."""
        assert W.dtype == np.float32 and I.dtype == np.int32 and W.flags.c_contiguous and I.flags.c_contiguous
        n1 = ctypes.c_int()
        n2 = ctypes.c_int()
        lib().orc_inq_quantize_weights(self._h, _fp(W), _ip(I), ctypes.byref(n1), ctypes.byref(n2))
        return n1.value, n2.value

    def commit(self, W, I):
        lib().orc_inq_commit(self._h, _fp(W), _ip(I))

    def affine(self, x, W, I, b=None):
        """Full INQAffine forward; W and I are updated in place; returns y."""
        x = _f32(x)
        M, K = x.shape
        N = W.size // K
        b = None if b is None else _f32(b)
        y = np.empty((M, N), np.float32)
        _check(lib().orc_inq_affine(self._h, _fp(x), _fp(W), _ip(I), _fp(b), _fp(y), ctypes.c_long(M),
                                    ctypes.c_long(K), ctypes.c_long(N)), "inq_affine")
        return y

    def convolution(self, x, W, I, b=None, pad=None, stride=None, dilation=None, group=1):
        x, _, tail, yshape = _conv_args(x, W, pad, stride, dilation, group)
        b = None if b is None else _f32(b)
        y = np.empty(yshape, np.float32)
        _check(lib().orc_inq_convolution(self._h, _fp(x), _fp(W), _ip(I), _fp(b), _fp(y), *tail), "inq_convolution")
        return y


class Bernoulli(object):
    """std::mt19937(seed) + std::bernoulli_distribution(0.5): the draw stream of INQ's random selection."""

    def __init__(self, seed):
        self._h = ctypes.c_void_p(lib().orc_bernoulli_create(int(seed)))

    def draw(self, count):
        out = np.empty(int(count), np.uint8)
        lib().orc_bernoulli_draw(self._h, out.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), ctypes.c_long(int(count)))
        return out

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_inq_destroy(self._h)
            self._h = None
