"""NNP / nntxt graph loading for the quantized-function path: ``NnpLoader`` with the reference's interface
(python/src/nnabla/utils/nnp_graph.py:84-135: ``get_network_names``, ``get_network(name, batch_size)`` ->
``NnpNetwork`` with ``variables`` / ``inputs`` / ``outputs``) plus the executor view of the C++ loader
(include/nbla_utils/nnp.hpp: ``get_executor`` -> data variables, output variables, ``execute``).

Functions are created through the registry for the *current* context, so a graph loaded under the ``hip`` extension
context runs on the hip:float classes (the dispatch nnp_impl_create_function.cpp.tmpl:51-117 performs for every
function; here for the nine quantization functions, QuantizeLinear, DequantizeLinear, Prune, Affine, ReLU, Add2, Sub2, Mul2, Div2 and
Concatenate).
Network definitions are read from protobuf text (``.nntxt`` / ``.prototxt``) or from binary protobuf
(``.protobuf``, load.py:492-494), parameters from ``parameter.protobuf`` or from ``parameter`` entries of either.
"""
import io
import os
import zipfile
from collections import OrderedDict

import numpy as np

from .. import functions as F
from ..variable import Variable
from . import nnp_format


class NnpError(ValueError):
    pass


def _shape_arg(p, name):
    s = p.get(name)
    return None if s is None else tuple(int(d) for d in s.all("dim"))


def _conv_kwargs(p):
    return dict(base_axis=int(p.get("base_axis", 1)), pad=_shape_arg(p, "pad"), stride=_shape_arg(p, "stride"),
                dilation=_shape_arg(p, "dilation"), group=int(p.get("group", 1)))


def _inq_kwargs(p):
    return dict(num_bits=int(p.get("num_bits", 4)), inq_iterations=tuple(int(i) for i in p.all("inq_iterations")),
                selection_algorithm=str(p.get("selection_algorithm", "largest_abs")), seed=int(p.get("seed", -1)))


def _opt(ins, i):
    return ins[i] if len(ins) > i else None


# type -> (name of the parameter message, number of required inputs, builder(param message, inputs) -> output).
# Argument names and defaults are those of functions.yaml:6735-7520.
_BUILDERS = {
    "FixedPointQuantize": ("fixed_point_quantize_param", 1, lambda p, i: F.fixed_point_quantize(
        i[0], sign=bool(p.get("sign", True)), n=int(p.get("n", 8)), delta=float(p.get("delta", 0.0625)),
        ste_fine_grained=bool(p.get("ste_fine_grained", True)))),
    "Pow2Quantize": ("pow2_quantize_param", 1, lambda p, i: F.pow2_quantize(
        i[0], sign=bool(p.get("sign", True)), with_zero=bool(p.get("with_zero", True)), n=int(p.get("n", 8)),
        m=int(p.get("m", 1)), ste_fine_grained=bool(p.get("ste_fine_grained", True)))),
    "MinMaxQuantize": ("min_max_quantize_param", 5, lambda p, i: F.min_max_quantize(
        i[0], i[1], i[2], i[3], i[4], decay=float(p.get("decay", 0.999)), x_min_max=bool(p.get("x_min_max", False)),
        ema=bool(p.get("ema", False)), ste_fine_grained=bool(p.get("ste_fine_grained", True)),
        eps=float(p.get("eps", 0.01)))),
    "BinaryWeightAffine": ("binary_weight_affine_param", 4, lambda p, i: F.binary_weight_affine(
        i[0], i[1], i[2], i[3], _opt(i, 4), base_axis=int(p.get("base_axis", 1)),
        quantize_zero_to=float(p.get("quantize_zero_to", 1.0)))),
    "BinaryConnectAffine": ("binary_connect_affine_param", 3, lambda p, i: F.binary_connect_affine(
        i[0], i[1], i[2], _opt(i, 3), base_axis=int(p.get("base_axis", 1)),
        quantize_zero_to=float(p.get("quantize_zero_to", 1.0)))),
    "BinaryWeightConvolution": ("binary_weight_convolution_param", 4, lambda p, i: F.binary_weight_convolution(
        i[0], i[1], i[2], i[3], _opt(i, 4), quantize_zero_to=float(p.get("quantize_zero_to", 1.0)),
        **_conv_kwargs(p))),
    "BinaryConnectConvolution": ("binary_connect_convolution_param", 3, lambda p, i: F.binary_connect_convolution(
        i[0], i[1], i[2], _opt(i, 3), quantize_zero_to=float(p.get("quantize_zero_to", 1.0)), **_conv_kwargs(p))),
    "INQAffine": ("inq_affine_param", 3, lambda p, i: F.inq_affine(
        i[0], i[1], i[2], _opt(i, 3), base_axis=int(p.get("base_axis", 1)), **_inq_kwargs(p))),
    "INQConvolution": ("inq_convolution_param", 3, lambda p, i: F.inq_convolution(
        i[0], i[1], i[2], _opt(i, 3), **dict(_conv_kwargs(p), **_inq_kwargs(p)))),
    "Affine": ("affine_param", 2, lambda p, i: F.affine(i[0], i[1], _opt(i, 2), base_axis=int(p.get("base_axis", 1)))),
    "Convolution": ("convolution_param", 2, lambda p, i: F.convolution(
        i[0], i[1], _opt(i, 2), channel_last=bool(p.get("channel_last", False)), **_conv_kwargs(p))),
    "ReLU": ("relu_param", 1, lambda p, i: F.relu(i[0], inplace=bool(p.get("inplace", False)))),
    "Add2": ("add2_param", 2, lambda p, i: F.add2(i[0], i[1], inplace=bool(p.get("inplace", False)))),
    "Sub2": ("sub2_param", 2, lambda p, i: F.sub2(i[0], i[1], inplace=bool(p.get("inplace", False)))),
    "Mul2": ("mul2_param", 2, lambda p, i: F.mul2(i[0], i[1], inplace=bool(p.get("inplace", False)))),
    "Div2": ("div2_param", 2, lambda p, i: F.div2(i[0], i[1], inplace=bool(p.get("inplace", False)))),
    "Pow2": ("pow2_param", 2, lambda p, i: F.pow2(i[0], i[1], inplace=bool(p.get("inplace", False)))),
    "Concatenate": ("concatenate_param", 2, lambda p, i: F.concatenate(
        *i, axis=int(p.get("axis", len(i[0].shape) - 1)))),
    "QuantizeLinear": ("quantize_linear_param", 3, lambda p, i: F.quantize_linear(
        i[0], i[1], i[2], round_mode=str(p.get("round_mode", "HALF_AWAY_FROM_ZERO")),
        narrow_range=bool(p.get("narrow_range", False)), dtype=int(p.get("dtype", 1)))),
    "DequantizeLinear": ("dequantize_linear_param", 3, lambda p, i: F.dequantize_linear(i[0], i[1], i[2])),
    "Prune": ("prune_param", 1, lambda p, i: F.prune(i[0], rate=float(p.get("rate", 0.9)))),
}

SUPPORTED_FUNCTIONS = tuple(sorted(_BUILDERS))


def _initial_value(var_msg, shape, rng):
    """Parameter without stored data: the variable's initializer (nnabla.proto.tmpl:100-103)."""
    init = var_msg.get("initializer")
    kind = str(init.get("type", "Constant")) if init is not None else "Constant"
    mult = float(init.get("multiplier", 0.0)) if init is not None else 0.0
    if kind == "Constant":
        return np.full(shape, mult, np.float32)
    if kind == "Normal":
        return (rng.randn(*shape) * mult).astype(np.float32)
    if kind == "Uniform":
        return rng.uniform(-mult, mult, size=shape).astype(np.float32)
    raise NnpError("initializer type %r is not supported (variable %r has no stored parameter)"
                   % (kind, var_msg.get("name")))


class NnpNetwork(object):
    """A variable graph built from one ``network`` message.

    ``variables``: every named variable; ``inputs``: Buffer variables no function produces; ``outputs``: variables
    no function consumes (nnp_graph.py:290-335)."""

    def __init__(self, net_msg, params, batch_size=None, rng=None):
        self.name = str(net_msg.get("name", ""))
        self.batch_size = int(batch_size if batch_size is not None else net_msg.get("batch_size", 1))
        if self.batch_size <= 0:
            raise NnpError("network %r: batch size must be positive" % self.name)
        rng = rng or np.random.RandomState(1223)
        self.variables = OrderedDict()
        declared = OrderedDict()
        for v in net_msg.all("variable"):
            name = str(v.get("name"))
            shape_msg = v.get("shape")
            dims = [int(d) for d in shape_msg.all("dim")] if shape_msg is not None else []
            shape = tuple(self.batch_size if d < 0 else d for d in dims)
            declared[name] = (str(v.get("type", "Buffer")), shape, v)
        produced, consumed = set(), set()
        for f in net_msg.all("function"):
            produced.update(str(o) for o in f.all("output"))
            consumed.update(str(i) for i in f.all("input"))
        for name, (kind, shape, msg) in declared.items():
            if kind == "Parameter":
                if name not in params:
                    params[name] = Variable.from_numpy_array(_initial_value(msg, shape, rng), need_grad=True)
                    params[name].name = name
                if tuple(params[name].shape) != shape:
                    raise NnpError("parameter %r: stored shape %s differs from the declared %s"
                                   % (name, tuple(params[name].shape), shape))
                self.variables[name] = params[name]
            elif name not in produced:
                v = Variable(shape)
                v.name = name
                self.variables[name] = v
        for f in net_msg.all("function"):
            self._add_function(f, declared)
        self.inputs = OrderedDict((n, v) for n, v in self.variables.items()
                                  if n in declared and declared[n][0] != "Parameter" and n not in produced)
        self.outputs = OrderedDict((n, v) for n, v in self.variables.items() if n in produced and n not in consumed)

    def _add_function(self, f, declared):
        ftype, fname = str(f.get("type")), str(f.get("name", ""))
        if ftype not in _BUILDERS:
            raise NnpError("function %r: type %r is not available on this path (supported: %s)"
                           % (fname, ftype, ", ".join(SUPPORTED_FUNCTIONS)))
        param_name, n_required, build = _BUILDERS[ftype]
        names = [str(i) for i in f.all("input")]
        if len(names) < n_required:
            raise NnpError("function %r (%s) needs at least %d inputs, got %d" % (fname, ftype, n_required, len(names)))
        missing = [n for n in names if n not in self.variables]
        if missing:
            raise NnpError("function %r reads undefined variable(s) %s" % (fname, missing))
        ins = [self.variables[n] for n in names]
        if ftype in ("INQAffine", "INQConvolution") and ins[2]._dtype(0) != np.dtype(np.int32):
            ins[2].set_data(ins[2].d, np.int32)  # stored parameters are float; the indicators are int (TI = int)
        outs = [str(o) for o in f.all("output")]
        if len(outs) != 1:
            raise NnpError("function %r (%s) must have exactly one output, got %d" % (fname, ftype, len(outs)))
        y = build(f.get(param_name) or nnp_format.Message(), ins)
        y.name = outs[0]
        if outs[0] in declared and declared[outs[0]][1] and tuple(y.shape) != declared[outs[0]][1]:
            raise NnpError("function %r: output %r has shape %s, the file declares %s"
                           % (fname, outs[0], tuple(y.shape), declared[outs[0]][1]))
        self.variables[outs[0]] = y


class NnpExecutor(object):
    """One ``executor`` message bound to its network (nnp.hpp: Executor)."""

    def __init__(self, exe_msg, network):
        self.name = str(exe_msg.get("name", ""))
        self.network = network
        self.data_variables = OrderedDict()
        for d in exe_msg.all("data_variable"):
            name = str(d.get("variable_name"))
            if name not in network.variables:
                raise NnpError("executor %r: data variable %r is not in network %r" % (self.name, name, network.name))
            self.data_variables[str(d.get("data_name", name))] = network.variables[name]
        self.output_variables = OrderedDict()
        for o in exe_msg.all("output_variable"):
            name = str(o.get("variable_name"))
            if name not in network.variables:
                raise NnpError("executor %r: output variable %r is not in network %r"
                               % (self.name, name, network.name))
            self.output_variables[str(o.get("data_name", name))] = network.variables[name]

    def execute(self):
        for v in self.output_variables.values():
            v.forward()


class NnpLoader(object):
    """Reads ``.nnp`` archives (zip of ``*.nntxt`` / ``*.prototxt`` and ``*.protobuf``) or a bare text file."""

    def __init__(self, filepath, scope=None, extension=".nntxt"):
        self._params = scope if scope is not None else OrderedDict()
        self._networks = OrderedDict()
        self._executors = OrderedDict()
        if hasattr(filepath, "read"):
            data, ext = filepath.read(), extension
        else:
            with open(filepath, "rb") as fh:
                data = fh.read()
            ext = os.path.splitext(filepath)[1]
        if ext == ".nnp":
            with zipfile.ZipFile(io.BytesIO(data)) as z:
                for name in z.namelist():
                    self._load_entry(name, z.read(name))
        else:
            self._load_entry("file" + ext, data)

    def _load_entry(self, name, data):
        ext = os.path.splitext(name)[1]
        if ext in (".nntxt", ".prototxt"):
            self._load_text(data.decode("utf-8") if isinstance(data, bytes) else data)
        elif ext == ".protobuf":
            # parameters, and (load.py:492-494) possibly the networks and executors as well
            for pname, (arr, need_grad) in nnp_format.decode_parameters(data).items():
                self._set_param(pname, arr, need_grad)
            self._register(nnp_format.decode_message(data, skip=("parameter",)))
        elif ext == ".h5":
            raise NnpError("%s: HDF5 parameter files are not supported here (h5py is absent); save the parameters "
                           "as parameter.protobuf" % name)
        # other entries (nnp_version.txt, ...) carry nothing the graph needs

    def _set_param(self, name, arr, need_grad):
        v = Variable.from_numpy_array(np.asarray(arr, np.float32), need_grad=bool(need_grad))
        v.name = name
        self._params[name] = v

    def _load_text(self, text):
        root = nnp_format.parse_text(text)
        for p in root.all("parameter"):
            shape_msg = p.get("shape")
            shape = tuple(int(d) for d in shape_msg.all("dim")) if shape_msg is not None else ()
            data = np.asarray([float(x) for x in p.all("data")], np.float32)
            if shape and data.size != int(np.prod(shape, dtype=np.int64)):
                raise NnpError("parameter %r: %d values for shape %s" % (p.get("variable_name"), data.size, shape))
            self._set_param(str(p.get("variable_name")), data.reshape(shape) if shape else data,
                            bool(p.get("need_grad", False)))
        self._register(root)

    def _register(self, root):
        for n in root.all("network"):
            self._networks[str(n.get("name"))] = n
        for e in root.all("executor"):
            self._executors[str(e.get("name"))] = e

    def get_network_names(self):
        return list(self._networks.keys())

    def get_network(self, name, batch_size=None, callback=None):
        if name not in self._networks:
            raise NnpError("no network named %r (have %s)" % (name, self.get_network_names()))
        return NnpNetwork(self._networks[name], self._params, batch_size)

    def get_executor_names(self):
        return list(self._executors.keys())

    def get_executor(self, name, batch_size=None):
        if name not in self._executors:
            raise NnpError("no executor named %r (have %s)" % (name, self.get_executor_names()))
        e = self._executors[name]
        return NnpExecutor(e, self.get_network(str(e.get("network_name")), batch_size))

    def get_parameters(self):
        return self._params


def save_nnp(path, nntxt, params):
    """Write an ``.nnp`` archive: the network text as ``network.nntxt`` and ``params`` (name -> array, or
    (array, need_grad)) as ``parameter.protobuf`` (the layout of nnabla.utils.save for ``.nnp`` targets)."""
    with zipfile.ZipFile(path, "w") as z:
        z.writestr("nnp_version.txt", "0.1\n")
        z.writestr("network.nntxt", nntxt)
        z.writestr("parameter.protobuf", nnp_format.encode_parameters(params))
