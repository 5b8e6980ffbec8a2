"""Variable and the minimal forward graph (mirrors the parts of python/src/nnabla/_variable.pyx and the graph engine
that the quantization functions need: ``.d`` / ``.g`` host access, ``.forward()``, ``.parent``, auto-forward)."""
import ctypes
from contextlib import contextmanager

import numpy as np

from . import _capi

# nbla::dtypes codes <-> numpy
_NP2DT = {np.dtype(np.bool_): 0, np.dtype(np.int8): 1, np.dtype(np.uint8): 2, np.dtype(np.int16): 3,
          np.dtype(np.uint16): 4, np.dtype(np.int32): 5, np.dtype(np.uint32): 6, np.dtype(np.int64): 7,
          np.dtype(np.uint64): 8, np.dtype(np.float32): 11, np.dtype(np.float64): 12}
_DT2NP = {v: k for k, v in _NP2DT.items()}
_DT2NP[9] = np.dtype(np.int64)
_DT2NP[10] = np.dtype(np.uint64)

_auto_forward = False


def get_auto_forward():
    return _auto_forward


def set_auto_forward(flag):
    global _auto_forward
    _auto_forward = bool(flag)


@contextmanager
def auto_forward(auto=True):
    """Functions execute as they are called (nnabla.auto_forward)."""
    global _auto_forward
    prev = _auto_forward
    _auto_forward = bool(auto)
    try:
        yield
    finally:
        _auto_forward = prev


def _shape_arr(shape):
    return (ctypes.c_int64 * len(shape))(*[int(s) for s in shape])


class NdArray(object):
    """The data (``which`` 0) or grad (``which`` 1) array of a variable: what ``v.data`` / ``v.grad`` return.  Passing
    one as ``outputs=[param.data]`` makes a function write its result into that array."""

    def __init__(self, var, which):
        self._var = var
        self._which = which

    @property
    def shape(self):
        return self._var.shape

    @property
    def data(self):
        return self._var._get(self._which)

    @data.setter
    def data(self, value):
        self._var._set(self._which, value)

    def zero(self):
        self._var._fill(self._which, 0.0)

    def fill(self, v):
        self._var._fill(self._which, v)


class Variable(object):
    """An N-d array with data and grad, living wherever it was last written (host or device)."""

    def __init__(self, shape=(), need_grad=False):
        L = _capi.lib()
        shape = tuple(int(s) for s in shape)
        self._h = _capi.check_handle(L.nblac_variable_new(_shape_arr(shape), len(shape)))
        self.need_grad = need_grad
        self.parent = None        # the FunctionNode that produces this variable
        self._consumers = []      # weak references to the FunctionNodes that take this variable as an input
        self._viewed = None       # the variable whose arrays this one views (set by reshape / unlink / rewire_on)
        self.name = ''
        self.persistent = False

    def __del__(self):
        h = getattr(self, "_h", None)
        if h and _capi._lib is not None:
            _capi._lib.nblac_variable_free(h)
            self._h = None

    @property
    def _origin(self):
        """The variable that owns the arrays this one views; itself for an ordinary variable (kept as None inside, so
        that a variable does not refer to itself and is freed as soon as it is dropped)."""
        return self if self._viewed is None else self._viewed

    @staticmethod
    def from_numpy_array(data, grad=None, need_grad=None):
        data = np.asarray(data)
        v = Variable(data.shape, need_grad=bool(need_grad))
        v._set(0, data, keep_dtype=True)
        if grad is not None:
            v._set(1, np.asarray(grad), keep_dtype=True)
        return v

    # ------------------------------------------------------------------ shape
    @property
    def shape(self):
        L = _capi.lib()
        nd = L.nblac_variable_ndim(self._h)
        out = (ctypes.c_int64 * max(nd, 1))()
        L.nblac_variable_shape(self._h, out)
        return tuple(int(out[i]) for i in range(nd))

    @property
    def ndim(self):
        return _capi.lib().nblac_variable_ndim(self._h)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def reset_shape(self, shape, force=False):
        _capi.check(_capi.lib().nblac_variable_reshape(self._h, _shape_arr(shape), len(shape), int(force)))

    def reshape(self, shape, unlink=False):
        """A variable sharing this one's arrays under another shape."""
        v = Variable(shape, self.need_grad)
        _capi.check(_capi.lib().nblac_variable_share(v._h, self._h))
        v._viewed = self._origin
        if not unlink:
            v.parent = self.parent
        return v

    # ------------------------------------------------------------- host access
    def _dtype(self, which):
        code = _capi.lib().nblac_variable_dtype(self._h, which)
        return _DT2NP.get(code, np.dtype(np.float32))

    def _get(self, which):
        dt = self._dtype(which)
        out = np.empty(self.shape, dt)
        _capi.check(_capi.lib().nblac_variable_get(self._h, which, out.ctypes.data_as(ctypes.c_void_p), _NP2DT[dt]))
        return out

    def _set(self, which, value, keep_dtype=False):
        value = np.asarray(value)
        # `.d = ...` keeps the array's current dtype (float32 for a fresh variable), as nnabla's setter does
        dt = value.dtype if keep_dtype and value.dtype in _NP2DT else self._dtype(which)
        arr = np.ascontiguousarray(np.broadcast_to(value, self.shape), dtype=dt)
        _capi.check(_capi.lib().nblac_variable_set(self._h, which, arr.ctypes.data_as(ctypes.c_void_p), _NP2DT[dt]))

    @property
    def data(self):
        return NdArray(self, 0)

    @property
    def grad(self):
        return NdArray(self, 1)

    def _share_array(self, other, which):
        """This variable's data or grad becomes a view of ``other``'s."""
        _capi.check(_capi.lib().nblac_variable_share_array(self._h, other._h, which))

    @property
    def d(self):
        """Data as a numpy array (a copy made through the host array class; device data is synchronised first)."""
        return self._get(0)

    @d.setter
    def d(self, value):
        self._set(0, value)

    @property
    def g(self):
        return self._get(1)

    @g.setter
    def g(self, value):
        self._set(1, value)

    def set_data(self, value, dtype=None):
        """Write with an explicit dtype (e.g. int32 indicators)."""
        value = np.asarray(value, dtype=dtype)
        self._set(0, value, keep_dtype=True)

    def zero(self):
        _capi.check(_capi.lib().nblac_variable_fill(self._h, 0, ctypes.c_double(0.0)))

    def fill(self, v):
        _capi.check(_capi.lib().nblac_variable_fill(self._h, 0, ctypes.c_double(float(v))))

    def _fill(self, which, v):
        _capi.check(_capi.lib().nblac_variable_fill(self._h, which, ctypes.c_double(float(v))))

    def zero_grad(self):
        self._fill(1, 0.0)

    @property
    def head_array_class(self):
        buf = ctypes.create_string_buffer(64)
        _capi.lib().nblac_variable_head_array_class(self._h, 0, buf, 64)
        return buf.value.decode()

    def device_pointer(self, dtype=np.float32, device_id='0'):
        """Raw device address of the data on a hip device (synchronises it there)."""
        p = _capi.lib().nblac_variable_device_pointer(self._h, 0, _NP2DT[np.dtype(dtype)], str(device_id).encode())
        if not p:
            _capi.check(_capi.lib().nblac_last_error_code() or 1)
        return p

    # ------------------------------------------------------------------- graph
    def _function_order(self):
        """The functions this variable depends on, each after the producers of its inputs."""
        done, order = set(), []
        stack = [(self.parent, 0)] if self.parent is not None else []
        if stack:
            done.add(id(self.parent))
        while stack:
            node, k = stack.pop()
            if k < len(node.inputs):
                stack.append((node, k + 1))
                nxt = node.inputs[k].parent
                if nxt is not None and id(nxt) not in done:
                    done.add(id(nxt))
                    stack.append((nxt, 0))
            else:
                order.append(node)
        return order

    def forward(self, clear_buffer=False, clear_no_need_grad=False):
        """Runs every function this variable depends on, in dependency order (CgVariable::forward)."""
        for node in self._function_order():
            node.forward()

    def visit(self, f):
        """Calls ``f(function)`` for every function this variable depends on, in forward order
        (python/src/nnabla/_variable.pyx, ``Variable.visit``)."""
        for node in self._function_order():
            f(node)

    @property
    def function_references(self):
        """The live functions that take this variable as an input, oldest first."""
        alive = [r for r in self._consumers if r() is not None]
        self._consumers = alive
        return [r() for r in alive]

    @property
    def rank(self):
        """0 for a leaf, else one more than the producing function's rank (function.cpp:109)."""
        ranks = {}
        for node in self._function_order():
            ranks[id(node)] = max([ranks.get(id(i.parent), -1) + 1 for i in node.inputs] or [0])
        return 0 if self.parent is None else ranks[id(self.parent)] + 1

    def rewire_on(self, var):
        """This variable takes over ``var``'s arrays and producing function, so that everything built on this variable
        now follows ``var``'s graph; ``var`` loses its parent (``Variable.rewire_on``, _variable.pyx:435-475)."""
        if tuple(var.shape) != tuple(self.shape):
            raise ValueError("rewire_on: shapes differ, %r and %r" % (self.shape, var.shape))
        _capi.check(_capi.lib().nblac_variable_share(self._h, var._h))
        self._viewed = var._origin
        node = var.parent
        self.parent = node
        if node is not None:
            node.outputs = [self if o is var else o for o in node.outputs]
            var.parent = None

    def backward(self, grad=1, clear_buffer=False):
        """Back-propagates from this variable (CgVariable::backward): its gradient is filled with `grad` (a scalar or an
        array; None keeps the current .g), then every function it depends on runs its backward in reverse order.
        Gradients of leaf variables are accumulated onto (zero them beforehand, as with nnabla); intermediate
        gradients are overwritten by their first contribution and accumulated by later ones."""
        if grad is not None:
            if np.isscalar(grad):
                self._fill(1, float(grad))
            else:
                self.g = np.asarray(grad)
        order = self._function_order()
        written = set()
        for node in reversed(order):
            if not any(i.need_grad for i in node.inputs):
                continue
            prop = [bool(i.need_grad) for i in node.inputs]
            # keyed by the variable that owns the grad array: two views of one array are one gradient, also when both
            # are inputs of this very function (its backward handles the inputs in order)
            accum = []
            for i, p in zip(node.inputs, prop):
                key = id(i._origin)
                accum.append((i.parent is None) or (key in written))
                if p:
                    written.add(key)
            node.backward(prop, accum)

    def get_unlinked_variable(self, need_grad=None):
        v = self.reshape(self.shape, unlink=True)
        v.need_grad = self.need_grad if need_grad is None else need_grad
        return v

    def __repr__(self):
        return "<Variable(%s, need_grad=%s)>" % (self.shape, self.need_grad)
