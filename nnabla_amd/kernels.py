"""ctypes binding of the kernel C-ABI (``include/nbla_hip_kernels.h``).

Device memory and streams come from the caller; the helpers at the bottom accept
``torch`` CUDA tensors purely as a convenient owner of device pointers.  Nothing
here computes on the host and nothing falls back to the CPU: a missing library or
a failing call raises ``KernelError``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnbla_hip_kernels.so")

OK = 0
ERR_NOT_IMPLEMENTED = -2
ERR_VALUE = -3
ERR_MEMORY = -5
ERR_RUNTIME = -10

#: every symbol declared in include/nbla_hip_kernels.h
EXPORTED = (
    "nbla_hip_init", "nbla_hip_last_error", "nbla_hip_version", "nbla_hip_cut_table",
    "nbla_hip_fixed_point_quantize_f32", "nbla_hip_pow2_quantize_f32",
    "nbla_hip_min_max_quantize_workspace_bytes", "nbla_hip_min_max_quantize_f32",
    "nbla_hip_min_max_quantize_static_f32",
    "nbla_hip_fixed_point_quantize_backward_f32", "nbla_hip_pow2_quantize_backward_f32",
    "nbla_hip_min_max_quantize_backward_workspace_bytes", "nbla_hip_min_max_quantize_backward_f32",
    "nbla_hip_packed_bits_bytes", "nbla_hip_digit_operand_bytes",
    "nbla_hip_binarize_workspace_bytes", "nbla_hip_binarize_weights_f32",
    "nbla_hip_split_digits_f32", "nbla_hip_gemm_bits_workspace_bytes", "nbla_hip_gemm_bits_f32",
    "nbla_hip_binary_affine_workspace_bytes", "nbla_hip_binary_weight_affine_f32",
    "nbla_hip_binary_connect_affine_f32", "nbla_hip_binary_affine_one_walk_f32", "nbla_hip_affine_f32", "nbla_hip_split_digits_scaled_f32",
    "nbla_hip_affine_workspace_bytes", "nbla_hip_affine_digits_f32",
    "nbla_hip_affine_backward_workspace_bytes", "nbla_hip_binary_affine_backward_f32", "nbla_hip_affine_backward_f32",
    "nbla_hip_convolution_output_shape", "nbla_hip_binary_convolution_workspace_bytes",
    "nbla_hip_binary_weight_convolution_f32", "nbla_hip_binary_connect_convolution_f32",
    "nbla_hip_convolution_backward_workspace_bytes", "nbla_hip_binary_convolution_backward_f32",
    "nbla_hip_convolution_backward_f32", "nbla_hip_convolution_workspace_bytes", "nbla_hip_convolution_f32",
    "nbla_hip_quantize_linear_f32", "nbla_hip_quantize_linear_backward_f32", "nbla_hip_dequantize_linear_f32",
    "nbla_hip_dequantize_linear_backward_f32", "nbla_hip_prune_workspace_bytes", "nbla_hip_prune_f32",
    "nbla_hip_range_recorder_workspace_bytes", "nbla_hip_range_recorder_f32",
    "nbla_hip_inq_workspace_bytes", "nbla_hip_inq_update_weights_f32", "nbla_hip_inq_affine_workspace_bytes",
    "nbla_hip_inq_affine_f32", "nbla_hip_inq_convolution_workspace_bytes", "nbla_hip_inq_convolution_f32",
    "nbla_hip_get_device_count", "nbla_hip_set_device", "nbla_hip_malloc", "nbla_hip_free", "nbla_hip_mem_info",
    "nbla_hip_memcpy", "nbla_hip_device_synchronize", "nbla_hip_stream_synchronize", "nbla_hip_fill",
    "nbla_hip_cast", "nbla_hip_relu_f32", "nbla_hip_relu_backward_f32", "nbla_hip_add2_f32",
    "nbla_hip_add2_backward_f32", "nbla_hip_binary2_f32", "nbla_hip_binary2_backward_f32", "nbla_hip_copy_rows_f32",
    "nbla_hip_broadcast2_f32", "nbla_hip_broadcast2_backward_workspace_bytes", "nbla_hip_broadcast2_backward_f32", "nbla_hip_mfma_rate_probe", "nbla_hip_binary_convolution_slab_plan",
    "nbla_hip_gemm_bits_timer_arm", "nbla_hip_gemm_bits_timer_read",
)


class KernelError(RuntimeError):
    def __init__(self, code, message):
        RuntimeError.__init__(self, "nbla_hip error %d: %s" % (code, message))
        self.code = code


_lib = None


def lib():
    """The loaded kernel library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KernelError(ERR_RUNTIME, "%s is missing: run `make -C nnabla_amd/csrc` (or "
                              "__graft_entry__.build())" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.nbla_hip_last_error.restype = ctypes.c_char_p
        L.nbla_hip_version.restype = ctypes.c_char_p
        for name in ("nbla_hip_min_max_quantize_workspace_bytes", "nbla_hip_packed_bits_bytes",
                     "nbla_hip_min_max_quantize_backward_workspace_bytes",
                     "nbla_hip_affine_backward_workspace_bytes",
                     "nbla_hip_convolution_backward_workspace_bytes", "nbla_hip_prune_workspace_bytes",
                     "nbla_hip_range_recorder_workspace_bytes", "nbla_hip_broadcast2_backward_workspace_bytes",
                     "nbla_hip_convolution_workspace_bytes", "nbla_hip_affine_workspace_bytes",
                     "nbla_hip_digit_operand_bytes", "nbla_hip_gemm_bits_workspace_bytes",
                     "nbla_hip_binarize_workspace_bytes",
                     "nbla_hip_binary_affine_workspace_bytes", "nbla_hip_binary_convolution_workspace_bytes",
                     "nbla_hip_inq_workspace_bytes", "nbla_hip_inq_affine_workspace_bytes",
                     "nbla_hip_inq_convolution_workspace_bytes"):
            getattr(L, name).restype = ctypes.c_size_t
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise KernelError(rc, lib().nbla_hip_last_error().decode())


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i64(v):
    return ctypes.c_int64(int(v))


def _shape(seq):
    return (ctypes.c_int64 * len(seq))(*[int(s) for s in seq])


def _stream(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(int(stream))


def _workspace(nbytes, like):
    import torch
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=like.device)


def init(device=0):
    check(lib().nbla_hip_init(int(device)))


def cut_table(which):
    out = (ctypes.c_uint32 * 277)()
    check(lib().nbla_hip_cut_table(int(which), out))
    return list(out)


# ------------------------------------------------------------------ tensor helpers

def fixed_point_quantize(x, sign=True, n=8, delta=2.0 ** -4, out=None, stream=None):
    import torch
    y = torch.empty_like(x) if out is None else out
    check(lib().nbla_hip_fixed_point_quantize_f32(_p(x), _p(y), ctypes.c_size_t(x.numel()), int(sign), int(n),
                                                  ctypes.c_float(delta), _stream(stream)))
    return y


def pow2_quantize(x, sign=True, with_zero=True, n=8, m=1, out=None, stream=None):
    import torch
    y = torch.empty_like(x) if out is None else out
    check(lib().nbla_hip_pow2_quantize_f32(_p(x), _p(y), ctypes.c_size_t(x.numel()), int(sign), int(with_zero),
                                           int(n), int(m), _stream(stream)))
    return y


def min_max_quantize(x, qr_min, qr_max, ql_min, ql_max, decay=0.999, x_min_max=False, ema=False, eps=0.01,
                     out=None, workspace=None, stream=None):
    """Updates qr_min / qr_max in place; returns (y, scale)."""
    import torch
    y = torch.empty_like(x) if out is None else out
    scale = torch.empty_like(qr_min)
    xs, qs = _shape(x.shape), _shape(qr_min.shape)
    need = lib().nbla_hip_min_max_quantize_workspace_bytes(xs, x.dim(), qs)
    ws = _workspace(need, x) if workspace is None else workspace
    check(lib().nbla_hip_min_max_quantize_f32(_p(x), _p(y), xs, x.dim(), qs, _p(qr_min), _p(qr_max), _p(ql_min),
                                              _p(ql_max), _p(scale), ctypes.c_float(decay), int(x_min_max), int(ema),
                                              ctypes.c_float(eps), _p(ws), ctypes.c_size_t(ws.numel()),
                                              _stream(stream)))
    return y, scale


def min_max_quantize_static(x, qr_min, qr_max, ql_min, ql_max, scale, y, decay=0.999, x_min_max=False, ema=False,
                            eps=0.01, stream=None):
    """The allocation-free variant: every buffer, outputs included, comes from the caller; the library's fixed
    per-device scratch replaces the workspace.  ``init(device)`` must have run."""
    xs, qs = _shape(x.shape), _shape(qr_min.shape)
    check(lib().nbla_hip_min_max_quantize_static_f32(_p(x), _p(y), xs, x.dim(), qs, _p(qr_min), _p(qr_max),
                                                     _p(ql_min), _p(ql_max), _p(scale), ctypes.c_float(decay),
                                                     int(x_min_max), int(ema), ctypes.c_float(eps), _stream(stream)))
    return y, scale


def _grad_out(dy, dx):
    import torch
    return (torch.empty_like(dy), 0) if dx is None else (dx, 1)


def fixed_point_quantize_backward(dy, x, sign=True, n=8, delta=2.0 ** -4, ste_fine_grained=True, dx=None,
                                  stream=None):
    """dx = STE gradient; a dx passed in is accumulated onto (in place)."""
    out, accum = _grad_out(dy, dx)
    check(lib().nbla_hip_fixed_point_quantize_backward_f32(_p(dy), _p(x), _p(out), ctypes.c_size_t(dy.numel()),
                                                           int(sign), int(n), ctypes.c_float(delta),
                                                           int(ste_fine_grained), accum, _stream(stream)))
    return out


def pow2_quantize_backward(dy, x, sign=True, with_zero=True, n=8, m=1, ste_fine_grained=True, dx=None, stream=None):
    out, accum = _grad_out(dy, dx)
    check(lib().nbla_hip_pow2_quantize_backward_f32(_p(dy), _p(x), _p(out), ctypes.c_size_t(dy.numel()), int(sign),
                                                    int(with_zero), int(n), int(m), int(ste_fine_grained), accum,
                                                    _stream(stream)))
    return out


def min_max_quantize_backward(dy, x, qr_min, qr_max, ql_min, ql_max, scale, ste_fine_grained=True, x_min_max=False,
                              ema=False, dx=None, g_qr_min=None, g_qr_max=None, want_x=True, want_min=True,
                              want_max=True, stream=None):
    """Returns (dx, g_qr_min, g_qr_max); gradients passed in are accumulated onto, None where not wanted."""
    import torch
    xs, qs = _shape(x.shape), _shape(qr_min.shape)
    ws = _workspace(lib().nbla_hip_min_max_quantize_backward_workspace_bytes(xs, x.dim(), qs), x)
    odx, ax = _grad_out(dy, dx) if want_x else (None, 0)
    omin, amin = _grad_out(qr_min, g_qr_min) if want_min else (None, 0)
    omax, amax = _grad_out(qr_max, g_qr_max) if want_max else (None, 0)
    check(lib().nbla_hip_min_max_quantize_backward_f32(
        _p(dy), _p(x), _p(odx), xs, x.dim(), qs, _p(qr_min), _p(qr_max), _p(ql_min), _p(ql_max), _p(scale), _p(omin),
        _p(omax), int(ste_fine_grained), int(x_min_max), int(ema), ax, amin, amax, _p(ws),
        ctypes.c_size_t(ws.numel()), _stream(stream)))
    return odx, omin, omax


def binarize_weights(W, K, N, transposed=False, quantize_zero_to=1.0, want_alpha=True, stream=None):
    """Returns (Wb, alpha or None, bits[uint32 tensor], zero_count tensor)."""
    import torch
    Wb = torch.empty_like(W)
    alpha = torch.empty(N, dtype=torch.float32, device=W.device) if want_alpha else None
    bits = torch.empty(lib().nbla_hip_packed_bits_bytes(_i64(K), _i64(N)) // 4, dtype=torch.int32, device=W.device)
    zc = torch.empty(1, dtype=torch.int32, device=W.device)
    ws = _workspace(lib().nbla_hip_binarize_workspace_bytes(_i64(K), _i64(N)), W)
    check(lib().nbla_hip_binarize_weights_f32(_p(W), _p(Wb), _p(alpha), _p(bits), _i64(K), _i64(N), int(transposed),
                                              ctypes.c_float(quantize_zero_to), _p(zc), _p(ws),
                                              ctypes.c_size_t(ws.numel()), _stream(stream)))
    return Wb, alpha, bits, zc


def split_digits(x, M, K, ldx=None, stream=None):
    """The int8 digit operand of x [M, K] (bytes): digit fragments, row sums, row shifts."""
    import torch
    out = torch.empty(lib().nbla_hip_digit_operand_bytes(_i64(M), _i64(K)), dtype=torch.uint8, device=x.device)
    check(lib().nbla_hip_split_digits_f32(_p(x), _i64(K if ldx is None else ldx), _p(out), _i64(M), _i64(K),
                                          _stream(stream)))
    return out


def gemm_bits(xsplit, bits, alpha, bias, M, K, N, out=None, inner=1, outer_stride=None, n_stride=1, workspace=None,
              stream=None):
    import torch
    y = torch.empty((M, N), dtype=torch.float32, device=bits.device) if out is None else out
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_gemm_bits_workspace_bytes(_i64(M), _i64(K), _i64(N)), bits)
    check(lib().nbla_hip_gemm_bits_f32(_p(xsplit), _p(bits), _p(alpha), _p(bias), _p(y), _i64(M), _i64(K), _i64(N),
                                       _i64(inner), _i64(N if outer_stride is None else outer_stride), _i64(n_stride),
                                       _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y


BROADCAST2_OPS = {"sub2": 0, "mul2": 1, "div2": 2, "add2": 3, "pow2": 4}


def broadcast2(op, x0, x1, stream=None):
    """y = op(x0, x1) with broadcasting (shapes of one rank, sizes equal or 1 along every axis)."""
    import torch
    shape = tuple(max(a, b) for a, b in zip(x0.shape, x1.shape))
    y = torch.empty(shape, dtype=torch.float32, device=x0.device)
    check(lib().nbla_hip_broadcast2_f32(BROADCAST2_OPS[op], _p(x0), _shape(x0.shape), _p(x1), _shape(x1.shape), _p(y),
                                        x0.dim(), _stream(stream)))
    return y


def broadcast2_backward(op, i, dy, x0, x1, dx=None, stream=None):
    """Gradient of input i; a dx passed in is accumulated onto (in place)."""
    import torch
    like = x0 if i == 0 else x1
    out, accum = (torch.empty_like(like), 0) if dx is None else (dx, 1)
    need = lib().nbla_hip_broadcast2_backward_workspace_bytes(int(i), _shape(x0.shape), _shape(x1.shape), x0.dim())
    ws = _workspace(need, dy) if need else None
    check(lib().nbla_hip_broadcast2_backward_f32(BROADCAST2_OPS[op], i, _p(dy), _p(x0), _shape(x0.shape), _p(x1),
                                                 _shape(x1.shape), _p(out), x0.dim(), accum, _p(ws),
                                                 ctypes.c_size_t(need), _stream(stream)))
    return out


def binary_affine_workspace(M, K, N, like):
    return _workspace(lib().nbla_hip_binary_affine_workspace_bytes(_i64(M), _i64(K), _i64(N)), like)


def binary_affine_one_walk(x, W, bias=None, quantize_zero_to=1.0, weight=True, workspace=None, stream=None):
    """The one-walk form of BinaryWeightAffine (weight=True) / BinaryConnectAffine: x [M,K], W [K,N] -> (y, Wb, alpha)."""
    import torch
    M, K = x.shape
    N = W.numel() // K
    Wb = torch.empty_like(W)
    alpha = torch.empty(N, dtype=torch.float32, device=x.device) if weight else None
    y = torch.empty((M, N), dtype=torch.float32, device=x.device)
    ws = binary_affine_workspace(M, K, N, x) if workspace is None else workspace
    check(lib().nbla_hip_binary_affine_one_walk_f32(_p(x), _p(W), _p(Wb), _p(alpha), _p(bias), _p(y), _i64(M), _i64(K),
                                                    _i64(N), ctypes.c_float(quantize_zero_to), _p(ws),
                                                    ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y, Wb, alpha


def binary_weight_affine(x, W, bias=None, quantize_zero_to=1.0, workspace=None, out=None, stream=None, Wb=None,
                         alpha=None):
    """x [M,K], W [K,N...] -> (y, Wb, alpha)."""
    import torch
    M, K = x.shape
    N = W.numel() // K
    Wb = torch.empty_like(W) if Wb is None else Wb
    alpha = torch.empty(N, dtype=torch.float32, device=x.device) if alpha is None else alpha
    y = torch.empty((M, N), dtype=torch.float32, device=x.device) if out is None else out
    ws = binary_affine_workspace(M, K, N, x) if workspace is None else workspace
    check(lib().nbla_hip_binary_weight_affine_f32(_p(x), _p(W), _p(Wb), _p(alpha), _p(bias), _p(y), _i64(M), _i64(K),
                                                  _i64(N), ctypes.c_float(quantize_zero_to), _p(ws),
                                                  ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y, Wb, alpha


def binary_connect_affine(x, W, bias=None, quantize_zero_to=1.0, workspace=None, out=None, stream=None, Wb=None):
    """x [M,K], W [K,N...] -> (y, Wb)."""
    import torch
    M, K = x.shape
    N = W.numel() // K
    Wb = torch.empty_like(W) if Wb is None else Wb
    y = torch.empty((M, N), dtype=torch.float32, device=x.device) if out is None else out
    ws = binary_affine_workspace(M, K, N, x) if workspace is None else workspace
    check(lib().nbla_hip_binary_connect_affine_f32(_p(x), _p(W), _p(Wb), _p(bias), _p(y), _i64(M), _i64(K), _i64(N),
                                                   ctypes.c_float(quantize_zero_to), _p(ws),
                                                   ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y, Wb


def _grads(shapes, given, want, like):
    import torch
    outs, accum = [], []
    for shp, g, w in zip(shapes, given, want):
        if not w:
            outs.append(None), accum.append(0)
        elif g is None:
            outs.append(torch.empty(shp, dtype=torch.float32, device=like.device)), accum.append(0)
        else:
            outs.append(g), accum.append(1)
    return outs, accum


def binary_affine_backward(dy, x, W, Wb=None, alpha=None, quantize_zero_to=1.0, dx=None, dW=None, db=None,
                           want=(True, True, True), workspace=None, stream=None):
    """(dx, dW, db) of BinaryWeightAffine (alpha given) / BinaryConnectAffine (alpha None); gradients passed in are
    accumulated onto in place."""
    M, K = x.shape
    N = W.numel() // K
    (odx, odw, odb), (ax, aw, ab) = _grads(((M, K), tuple(W.shape), (N,)), (dx, dW, db), want, x)
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_affine_backward_workspace_bytes(_i64(M), _i64(K), _i64(N)), x)
    check(lib().nbla_hip_binary_affine_backward_f32(_p(dy), _p(x), _p(W), _p(Wb), _p(alpha), _p(odx), _p(odw), _p(odb),
                                                    _i64(M), _i64(K), _i64(N), ctypes.c_float(quantize_zero_to), ax,
                                                    aw, ab, _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return odx, odw, odb


def affine_backward(dy, x, W, dx=None, dW=None, db=None, want=(True, True, True), workspace=None, stream=None):
    """(dx, dW, db) of y = x.W + b with real-valued weights."""
    M, K = x.shape
    N = W.numel() // K
    (odx, odw, odb), (ax, aw, ab) = _grads(((M, K), tuple(W.shape), (N,)), (dx, dW, db), want, x)
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_affine_backward_workspace_bytes(_i64(M), _i64(K), _i64(N)), x)
    check(lib().nbla_hip_affine_backward_f32(_p(dy), _p(x), _p(W), _p(odx), _p(odw), _p(odb), _i64(M), _i64(K), _i64(N),
                                             ax, aw, ab, _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return odx, odw, odb


def affine_digits(x, W, bias=None, out=None, workspace=None, stream=None):
    """y = x.W + b on the int8 digit kernels."""
    import torch
    M, K = x.shape
    N = W.numel() // K
    y = torch.empty((M, N), dtype=torch.float32, device=x.device) if out is None else out
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_affine_workspace_bytes(_i64(M), _i64(K), _i64(N)), x)
    check(lib().nbla_hip_affine_digits_f32(_p(x), _p(W), _p(bias), _p(y), _i64(M), _i64(K), _i64(N), _p(ws),
                                           ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y


def affine(x, W, bias=None, out=None, stream=None):
    import torch
    M, K = x.shape
    N = W.numel() // K
    y = torch.empty((M, N), dtype=torch.float32, device=x.device) if out is None else out
    check(lib().nbla_hip_affine_f32(_p(x), _p(W), _p(bias), _p(y), _i64(M), _i64(K), _i64(N), _stream(stream)))
    return y


def _conv_geometry(x, W, pad, stride, dilation, group):
    nd = W.dim() - 2
    outer = 1
    for s in x.shape[:x.dim() - nd - 1]:
        outer *= int(s)
    C = int(x.shape[x.dim() - nd - 1])
    in_sp = [int(s) for s in x.shape[x.dim() - nd:]]
    O = int(W.shape[0])
    kernel = [int(s) for s in W.shape[2:]]
    pad = list(pad) if pad is not None else [0] * nd
    stride = list(stride) if stride is not None else [1] * nd
    dilation = list(dilation) if dilation is not None else [1] * nd
    out_sp = (ctypes.c_int64 * nd)()
    check(lib().nbla_hip_convolution_output_shape(nd, _shape(in_sp), _shape(kernel), _shape(pad), _shape(stride),
                                                  _shape(dilation), out_sp))
    geom = (_i64(outer), _i64(C), nd, _shape(in_sp), _i64(O), _shape(kernel), _shape(pad), _shape(stride),
            _shape(dilation), _i64(group))
    yshape = tuple(x.shape[:x.dim() - nd - 1]) + (O,) + tuple(int(v) for v in out_sp)
    return geom, yshape


def binary_weight_convolution(x, W, bias=None, pad=None, stride=None, dilation=None, group=1, quantize_zero_to=1.0,
                              stream=None):
    """x [..., C, spatial...], W [O, C/group, kernel...] -> (y, Wb, alpha)."""
    import torch
    geom, yshape = _conv_geometry(x, W, pad, stride, dilation, group)
    q0 = ctypes.c_float(quantize_zero_to)
    ws = _workspace(lib().nbla_hip_binary_convolution_workspace_bytes(*geom, q0), x)
    Wb = torch.empty_like(W)
    alpha = torch.empty(W.shape[0], dtype=torch.float32, device=x.device)
    y = torch.empty(yshape, dtype=torch.float32, device=x.device)
    check(lib().nbla_hip_binary_weight_convolution_f32(_p(x), _p(W), _p(Wb), _p(alpha), _p(bias), _p(y), *geom, q0,
                                                       _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y, Wb, alpha


def binary_convolution_slab_plan(outer, C, in_sp, O, kernel, pad, stride, dilation, group=1):
    """The host's plan for a binary convolution that keeps a block's input positions in LDS: a dict with the output
    positions per block, blocks per sample, input positions held and LDS bytes, or None where the geometry takes
    the gathering product.  Shapes only; touches no device."""
    plan = (ctypes.c_int32 * 4)()
    check(lib().nbla_hip_binary_convolution_slab_plan(
        _i64(outer), _i64(C), ctypes.c_int(len(in_sp)), _shape(in_sp), _i64(O), _shape(kernel), _shape(pad),
        _shape(stride), _shape(dilation), _i64(group), plan))
    if plan[0] == 0:
        return None
    return {"tile_rows": plan[0], "tiles_per_sample": plan[1], "cap": plan[2], "lds_bytes": plan[3]}


def binary_connect_convolution(x, W, bias=None, pad=None, stride=None, dilation=None, group=1, quantize_zero_to=1.0,
                               stream=None):
    """x [..., C, spatial...], W [O, C/group, kernel...] -> (y, Wb)."""
    import torch
    geom, yshape = _conv_geometry(x, W, pad, stride, dilation, group)
    q0 = ctypes.c_float(quantize_zero_to)
    ws = _workspace(lib().nbla_hip_binary_convolution_workspace_bytes(*geom, q0), x)
    Wb = torch.empty_like(W)
    y = torch.empty(yshape, dtype=torch.float32, device=x.device)
    check(lib().nbla_hip_binary_connect_convolution_f32(_p(x), _p(W), _p(Wb), _p(bias), _p(y), *geom, q0, _p(ws),
                                                        ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y, Wb


def binary_convolution_backward(dy, x, W, Wb=None, alpha=None, pad=None, stride=None, dilation=None, group=1,
                                quantize_zero_to=1.0, dx=None, dW=None, db=None, want=(True, True, True),
                                workspace=None, stream=None):
    """(dx, dW, db) of BinaryWeightConvolution (alpha given) / BinaryConnectConvolution (alpha None); gradients
    passed in are accumulated onto in place."""
    geom, _ = _conv_geometry(x, W, pad, stride, dilation, group)
    (odx, odw, odb), (ax, aw, ab) = _grads((tuple(x.shape), tuple(W.shape), (int(W.shape[0]),)), (dx, dW, db), want, x)
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_convolution_backward_workspace_bytes(*geom), x)
    check(lib().nbla_hip_binary_convolution_backward_f32(_p(dy), _p(x), _p(W), _p(Wb), _p(alpha), _p(odx), _p(odw),
                                                         _p(odb), *geom, ctypes.c_float(quantize_zero_to), ax, aw, ab,
                                                         _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return odx, odw, odb


def convolution_backward(dy, x, W, pad=None, stride=None, dilation=None, group=1, dx=None, dW=None, db=None,
                         want=(True, True, True), workspace=None, stream=None):
    """(dx, dW, db) of a convolution with real-valued weights."""
    geom, _ = _conv_geometry(x, W, pad, stride, dilation, group)
    (odx, odw, odb), (ax, aw, ab) = _grads((tuple(x.shape), tuple(W.shape), (int(W.shape[0]),)), (dx, dW, db), want, x)
    ws = workspace if workspace is not None else _workspace(
        lib().nbla_hip_convolution_backward_workspace_bytes(*geom), x)
    check(lib().nbla_hip_convolution_backward_f32(_p(dy), _p(x), _p(W), _p(odx), _p(odw), _p(odb), *geom, ax, aw, ab,
                                                  _p(ws), ctypes.c_size_t(ws.numel()), _stream(stream)))
    return odx, odw, odb


# ------------------------------------------------------- QuantizeLinear / DequantizeLinear / Prune

DTYPE_BYTE, DTYPE_UBYTE = 1, 2


def quantize_linear(x, scale, zero_point, round_mode="HALF_AWAY_FROM_ZERO", narrow_range=False, dtype=DTYPE_BYTE,
                    stream=None):
    """y = saturate(round(x / scale) + zero_point); ``zero_point`` is rounded and saturated in place."""
    import torch
    y = torch.empty_like(x)
    check(lib().nbla_hip_quantize_linear_f32(_p(x), _p(scale), _p(zero_point), _p(y), _shape(x.shape),
                                             _shape(scale.shape), _shape(zero_point.shape), x.dim(),
                                             int(round_mode == "HALF_TO_EVEN"), int(narrow_range), int(dtype),
                                             _stream(stream)))
    return y


def dequantize_linear(x, scale, zero_point, stream=None):
    import torch
    y = torch.empty_like(x)
    check(lib().nbla_hip_dequantize_linear_f32(_p(x), _p(scale), _p(zero_point), _p(y), _shape(x.shape),
                                               _shape(scale.shape), _shape(zero_point.shape), x.dim(),
                                               _stream(stream)))
    return y


def linear_quantize_backward(dy, scale, dequantize=False, dx=None, stream=None):
    """dx (+)= dy / scale (QuantizeLinear) or dy * scale (DequantizeLinear)."""
    out, accum = _grad_out(dy, dx)
    fn = lib().nbla_hip_dequantize_linear_backward_f32 if dequantize else lib().nbla_hip_quantize_linear_backward_f32
    check(fn(_p(dy), _p(scale), _p(out), _shape(dy.shape), _shape(scale.shape), dy.dim(), accum, _stream(stream)))
    return out


def prune(x, rate=0.9, workspace=None, stream=None):
    import torch
    y = torch.empty_like(x)
    ws = workspace if workspace is not None else _workspace(lib().nbla_hip_prune_workspace_bytes(), x)
    check(lib().nbla_hip_prune_f32(_p(x), _p(y), ctypes.c_size_t(x.numel()), ctypes.c_float(rate), _p(ws),
                                   ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y


RECORDER_MODES = {"MinMaxMinMaxRecorder": 0, "AbsMaxRecorder": 1, "MinMaxMvaRecorder": 2, "MaxMaxRecorder": 3,
                  "MaxMvaRecorder": 4}


def range_recorder(x, m, M, mode, decay=0.99, training=True, y=None, workspace=None, stream=None):
    """y = x; m / M (one-element tensors, updated in place; m may be None for the one-sided recorders) take this
    batch's statistics.  `mode` is a key or value of RECORDER_MODES."""
    import torch
    mode = RECORDER_MODES.get(mode, mode)
    y = torch.empty_like(x) if y is None else y
    ws = workspace if workspace is not None else _workspace(lib().nbla_hip_range_recorder_workspace_bytes(), x)
    check(lib().nbla_hip_range_recorder_f32(_p(x), _p(y), ctypes.c_size_t(x.numel()), _p(m) if m is not None else None,
                                            _p(M), int(mode), ctypes.c_double(decay), int(bool(training)), _p(ws),
                                            ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y


# ---------------------------------------------------------------------------- INQ

INQ_PRODUCT_ONLY, INQ_NO_SELECTION, INQ_FIX_ALL, INQ_LARGEST_ABS, INQ_RANDOM = -1, 0, 1, 2, 3
BERNOULLI_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint8), ctypes.c_int64)


def _draw_callback(draw):
    """Wraps a Python callable count -> sequence of 0/1 as the C callback of step 3."""
    if draw is None:
        return ctypes.cast(None, BERNOULLI_FN)

    def cb(_ctx, out, count):
        vals = draw(int(count))
        for i in range(int(count)):
            out[i] = int(vals[i])
    return BERNOULLI_FN(cb)


def inq_update_weights(W, I, old_W, old_I, num_bits, step, draw=None, stream=None):
    """Steps A-C and F in place on W (fp32) and I (int32); returns a device tensor (n1, n2)."""
    import torch
    size = W.numel()
    ws = _workspace(lib().nbla_hip_inq_workspace_bytes(_i64(size), int(step)), W)
    n1n2 = torch.empty(2, dtype=torch.int32, device=W.device)
    cb = _draw_callback(draw)
    check(lib().nbla_hip_inq_update_weights_f32(_p(W), _p(I), _p(old_W), _p(old_I), _i64(size), int(num_bits),
                                                int(step), cb, None, _p(n1n2), _p(ws), ctypes.c_size_t(ws.numel()),
                                                _stream(stream)))
    return n1n2


def inq_affine(x, W, I, old_W, old_I, bias=None, num_bits=4, step=0, draw=None, stream=None):
    """INQAffine forward; W, I, old_W, old_I are updated in place; returns y."""
    import torch
    M, K = x.shape
    N = W.numel() // K
    ws = _workspace(lib().nbla_hip_inq_affine_workspace_bytes(_i64(M), _i64(K), _i64(N), int(step)), x)
    y = torch.empty((M, N), dtype=torch.float32, device=x.device)
    cb = _draw_callback(draw)
    check(lib().nbla_hip_inq_affine_f32(_p(x), _p(W), _p(I), _p(old_W), _p(old_I), _p(bias), _p(y), _i64(M), _i64(K),
                                        _i64(N), int(num_bits), int(step), cb, None, _p(ws),
                                        ctypes.c_size_t(ws.numel()), _stream(stream)))
    return y


def inq_convolution(x, W, I, old_W, old_I, bias=None, pad=None, stride=None, dilation=None, group=1, num_bits=4,
                    step=0, draw=None, stream=None):
    import torch
    geom, yshape = _conv_geometry(x, W, pad, stride, dilation, group)
    ws = _workspace(lib().nbla_hip_inq_convolution_workspace_bytes(*geom, int(step)), x)
    y = torch.empty(yshape, dtype=torch.float32, device=x.device)
    cb = _draw_callback(draw)
    check(lib().nbla_hip_inq_convolution_f32(_p(x), _p(W), _p(I), _p(old_W), _p(old_I), _p(bias), _p(y), *geom,
                                             int(num_bits), int(step), cb, None, _p(ws), ctypes.c_size_t(ws.numel()),
                                             _stream(stream)))
    return y


def gemm_bits_timer_arm(launches):
    """The calling thread's next `launches` launches of the bit-weight product record their own begin and end."""
    check(lib().nbla_hip_gemm_bits_timer_arm(ctypes.c_int(int(launches))))


def gemm_bits_timer_read():
    """Waits for the armed launches made so far; {launches, mean_ms, min_ms, max_ms} of the kernel itself."""
    n = ctypes.c_int(0)
    mean, lo, hi = ctypes.c_double(0.0), ctypes.c_double(0.0), ctypes.c_double(0.0)
    check(lib().nbla_hip_gemm_bits_timer_read(ctypes.byref(n), ctypes.byref(mean), ctypes.byref(lo), ctypes.byref(hi)))
    return {"launches": n.value, "mean_ms": mean.value, "min_ms": lo.value, "max_ms": hi.value}


MFMA_PROBE_KINDS = {"i8": 0, "fp6 x fp4": 1, "fp8 x fp8": 2, "i8, operands change": 3,
                    "i8, digits x bit bytes, operands change": 4}


def mfma_rate_probe(kind, rounds, sink, stream=None):
    """Launches the matrix-instruction rate probe (measurement utility of bench.py); returns (instructions issued,
    operations per instruction).  `sink`: a float tensor on the device (never written)."""
    n, ops = ctypes.c_int64(0), ctypes.c_int64(0)
    check(lib().nbla_hip_mfma_rate_probe(ctypes.c_int(MFMA_PROBE_KINDS[kind]), ctypes.c_int(int(rounds)),
                                         ctypes.byref(n), ctypes.byref(ops), _p(sink), _stream(stream)))
    return n.value, ops.value
