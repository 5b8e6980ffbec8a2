"""Function objects and graph nodes (the subset of python/src/nnabla/function.pyx.tmpl the path needs)."""
import ctypes
import weakref

from . import _capi
from .context import get_current_context
from .variable import NdArray, Variable, get_auto_forward


def _handles(variables):
    return (ctypes.c_void_p * len(variables))(*[v._h for v in variables])


class Info(dict):
    """What a function was created from: the registry name with the packed integer / float / string arguments (the
    dict items), plus ``type_name`` (the name the function reports, as ``nnabla.function.Info.type_name``) and
    ``args`` (the keyword arguments of the ``F.*`` call, as ``Info.args``)."""

    def __init__(self, name, iargs, fargs, sarg, args=None, type_name=None):
        dict.__init__(self, type=name, iargs=tuple(iargs), fargs=tuple(fargs), sarg=sarg)
        self.args = dict(args or {})
        self.type_name = type_name or name


class Function(object):
    """A function instance created through the nbla registry for the current (or given) context."""

    def __init__(self, name, ctx=None, iargs=(), fargs=(), sarg=None, args=None):
        L = _capi.lib()
        ctx = ctx or get_current_context()
        self.ctx = ctx
        backends = (ctypes.c_char_p * len(ctx.backend))(*[b.encode() for b in ctx.backend])
        ia = (ctypes.c_int64 * max(1, len(iargs)))(*[int(i) for i in iargs])
        fa = (ctypes.c_double * max(1, len(fargs)))(*[float(f) for f in fargs])
        h = L.nblac_function_create(name.encode(), backends, len(ctx.backend), ctx.array_class.encode(),
                                    str(ctx.device_id).encode(), ia, len(iargs), fa, len(fargs),
                                    None if sarg is None else sarg.encode())
        self._h = _capi.check_handle(h)
        self.info = Info(name, iargs, fargs, sarg, args)
        if name == "RangeRecorder":
            self.info.type_name = self.name

    def clone(self, ctx=None):
        """A new function of the same type and arguments (what the graph converters' ``_modify_as_same`` builds by
        evaluating ``F.<type_name>(ctx, **args)``, graph_converter.py:138-151)."""
        i = self.info
        return Function(i["type"], ctx, i["iargs"], i["fargs"], i["sarg"], i.args)

    def __del__(self):
        h = getattr(self, "_h", None)
        if h and _capi._lib is not None:
            _capi._lib.nblac_function_free(h)
            self._h = None

    @property
    def name(self):
        buf = ctypes.create_string_buffer(128)
        _capi.lib().nblac_function_name(self._h, buf, 128)
        return buf.value.decode()

    @property
    def min_outputs(self):
        return _capi.lib().nblac_function_min_outputs(self._h)

    def setup(self, inputs, outputs):
        _capi.check(_capi.lib().nblac_function_setup(self._h, _handles(inputs), len(inputs), _handles(outputs),
                                                     len(outputs)))

    def forward(self, inputs, outputs):
        _capi.check(_capi.lib().nblac_function_forward(self._h, _handles(inputs), len(inputs), _handles(outputs),
                                                       len(outputs)))

    def recompute(self, inputs, outputs):
        _capi.check(_capi.lib().nblac_function_recompute(self._h, _handles(inputs), len(inputs), _handles(outputs),
                                                         len(outputs)))

    def backward(self, inputs, outputs, propagate_down=None, accum=None):
        """Function::backward: gradients of the outputs (their .g) -> gradients of the inputs flagged in
        propagate_down, added to the existing ones where accum is set."""
        n = len(inputs)
        prop = [True] * n if propagate_down is None else list(propagate_down)
        acc = [False] * n if accum is None else list(accum)
        flags = (ctypes.c_ubyte * max(1, n))(*[(1 if prop[i] else 0) | (2 if acc[i] else 0) for i in range(n)])
        _capi.check(_capi.lib().nblac_function_backward_flags(self._h, _handles(inputs), n, _handles(outputs),
                                                              len(outputs), flags))

    def __call__(self, *inputs, **kw):
        """Connects the function to its inputs: creates outputs, runs setup (shape inference), executes at once in
        auto-forward mode (function.pyx.tmpl:309-344)."""
        outputs = kw.get("outputs")
        n_outputs = kw.get("n_outputs", -1)
        inputs = list(inputs)
        n = self.min_outputs if n_outputs < 0 else n_outputs
        outs = []
        for i in range(n):
            given = outputs[i] if outputs is not None and i < len(outputs) else None
            if isinstance(given, NdArray):
                # a fresh output variable writing into the given array (function.pyx.tmpl:318-326)
                v = Variable(given.shape)
                v._share_array(given._var, given._which)
                outs.append(v)
            elif given is not None:
                outs.append(given)
            else:
                outs.append(Variable(()))
        self.setup(inputs, outs)
        node = FunctionNode(self, inputs, outs)
        for o in outs:
            o.parent = node
            o.need_grad = any(i.need_grad for i in inputs)
        if get_auto_forward():
            node.forward()
        return outs[0] if len(outs) == 1 else tuple(outs)


class FunctionNode(object):
    """A function bound to its input and output variables (CgFunction)."""

    def __init__(self, function, inputs, outputs):
        self.function = function
        self.inputs = inputs
        self.outputs = outputs
        ref = weakref.ref(self)
        for v in {id(i): i for i in inputs}.values():
            v._consumers.append(ref)

    @property
    def rank(self):
        """Longest path from a leaf variable (CgFunction::rank, computation_graph.cpp:28-35)."""
        return max([i.rank for i in self.inputs] or [0])

    @property
    def name(self):
        return self.function.name

    @property
    def info(self):
        return self.function.info

    def forward(self):
        self.function.forward(self.inputs, self.outputs)

    def recompute(self):
        self.function.recompute(self.inputs, self.outputs)

    def backward(self, propagate_down, accum):
        self.function.backward(self.inputs, self.outputs, propagate_down, accum)
