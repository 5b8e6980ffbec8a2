"""Writing a graph as an NNP file (the network / executor part of python/src/nnabla/utils/save.py:75-84,241-287,
289-470): what ``nnabla_amd.utils.nnp_graph.NnpLoader`` -- and nnabla's own loaders -- read back.

``contents`` follows the reference::

    {'networks':  [{'name': 'net', 'batch_size': 16, 'outputs': {'y': y}, 'names': {'x': x}}],
     'executors': [{'name': 'runtime', 'network': 'net', 'data': ['x'], 'output': ['y']}]}

Optimizers, monitors, datasets and training configurations are not written (there is no solver on this path);
parameters go into ``parameter.protobuf`` (HDF5 needs h5py, which is absent).
"""
import io
import os
import zipfile
from collections import OrderedDict

from .. import parameter
from . import nnp_format
from .nnp_format import Message
from .nnp_graph import _BUILDERS

_SHAPE_FIELDS = ("pad", "stride", "dilation")
_LIST_FIELDS = ("inq_iterations",)


def _same_arrays(a, b):
    return a._origin is b._origin and tuple(a.shape) == tuple(b.shape)


def _shape_message(shape, batch_size=None):
    m = Message()
    for k, d in enumerate(shape):
        m.add("dim", -1 if (k == 0 and batch_size is not None and d == batch_size) else int(d))
    return m


def _function_param(info):
    """The ``<type>_param`` message of a function from the keyword arguments it was created with."""
    m = Message()
    for key, val in info.args.items():
        if key in _SHAPE_FIELDS:
            m.add(key, _shape_message(val))
        elif key in _LIST_FIELDS:
            for v in val:
                m.add(key, int(v))
        elif isinstance(val, (bool, int, float, str)):
            m.add(key, val)
        else:
            m.add(key, float(val))
    return m


def _ordered_functions(outputs):
    seen, order = set(), []
    for v in outputs:
        for f in v._function_order():
            if id(f) not in seen:
                seen.add(id(f))
                order.append(f)
    return order


def _network_message(net, variable_batch_size, used_params):
    name = net['name']
    batch_size = int(net.get('batch_size', 1))
    outputs = OrderedDict(net['outputs'])
    given = OrderedDict(net.get('names', {}))
    given.update(outputs)
    registered = parameter.get_parameters(grad_only=False)
    functions = _ordered_functions(list(outputs.values()))

    names = {}                 # id(variable of the graph) -> name
    kinds = OrderedDict()      # name -> (kind, variable)

    def name_of(v, fallback):
        if id(v) in names:
            return names[id(v)]
        for n, u in given.items():
            if u is v or (v.parent is None and u.parent is None and _same_arrays(u, v)):
                chosen, kind = n, "Buffer"
                break
        else:
            for n, u in registered.items():
                if u is v or (v.parent is None and _same_arrays(u, v)):
                    chosen, kind = n, "Parameter"
                    used_params[n] = u
                    break
            else:
                chosen, kind = fallback, "Buffer"
        if chosen in kinds and kinds[chosen][1] is not v and not _same_arrays(kinds[chosen][1], v):
            raise ValueError("network %r: two different variables would be named %r" % (name, chosen))
        names[id(v)] = chosen
        kinds.setdefault(chosen, (kind, v))
        return chosen

    msg = Message()
    msg.add("name", name)
    msg.add("batch_size", batch_size)
    fmsgs, n_inputs = [], 0
    for k, f in enumerate(functions):
        ftype = f.info.type_name
        if ftype not in _BUILDERS:
            raise ValueError("network %r: function type %r cannot be stored in an NNP file" % (name, ftype))
        fm = Message()
        fm.add("name", "%s_%d" % (ftype, k))
        fm.add("type", ftype)
        for v in f.inputs:
            if v.parent is None and id(v) not in names:
                n_inputs += 1
            fm.add("input", name_of(v, "Input_%d" % n_inputs))
        for j, v in enumerate(f.outputs):
            fm.add("output", name_of(v, "%s_%d_Output%s" % (ftype, k, "" if j == 0 else "_%d" % j)))
        if f.info.args:
            fm.add(_BUILDERS[ftype][0], _function_param(f.info))
        fmsgs.append(fm)
    for n, (kind, v) in kinds.items():
        vm = Message()
        vm.add("name", n)
        vm.add("type", kind)
        vm.add("shape", _shape_message(v.shape, batch_size if (variable_batch_size and kind == "Buffer") else None))
        msg.add("variable", vm)
    for fm in fmsgs:
        msg.add("function", fm)
    return msg, set(kinds), [n for n, (kind, _) in kinds.items() if kind == "Parameter"]


def _executor_message(exe, network_variables, network_parameters):
    m = Message()
    m.add("name", exe['name'])
    m.add("network_name", exe['network'])
    outs = exe.get('output', exe.get('outputs', []))
    for key, field in ((exe.get('data', []), "data_variable"), (outs, "output_variable")):
        for n in key:
            if n not in network_variables:
                raise ValueError("executor %r: %r is not a variable of network %r" % (exe['name'], n, exe['network']))
            d = Message()
            d.add("variable_name", n)
            d.add("data_name", n)
            m.add(field, d)
    for n in network_parameters:
        d = Message()
        d.add("variable_name", n)
        m.add("parameter_variable", d)
    return m


def create_proto(contents, include_params=False, variable_batch_size=True):
    """(root message, {parameter name: variable}) for ``contents``."""
    unsupported = [k for k in ('optimizers', 'monitors', 'datasets', 'training_config') if contents.get(k)]
    if unsupported:
        raise NotImplementedError("save: %s are not written by this package" % ", ".join(unsupported))
    root = Message()
    used = OrderedDict()
    nets = {}
    for net in contents.get('networks', []):
        msg, variables, params = _network_message(net, variable_batch_size, used)
        nets[net['name']] = (variables, params)
        root.add("network", msg)
    for exe in contents.get('executors', []):
        if exe['network'] not in nets:
            raise ValueError("executor %r refers to unknown network %r" % (exe['name'], exe['network']))
        root.add("executor", _executor_message(exe, *nets[exe['network']]))
    if include_params:
        for n, v in used.items():
            pm = Message()
            pm.add("variable_name", n)
            pm.add("shape", _shape_message(v.shape))
            for x in v.d.ravel().tolist():
                pm.add("data", float(x))
            pm.add("need_grad", bool(v.need_grad))
            root.add("parameter", pm)
    return root, used


def save(filename, contents, include_params=False, variable_batch_size=True, extension=".nnp", parameters=None,
         parameter_format=".protobuf"):
    """Write ``contents`` to ``filename`` (a path or a file object; then ``extension`` names the format): ``.nnp`` --
    a zip of ``nnp_version.txt``, ``network.nntxt`` and ``parameter.protobuf`` -- or ``.nntxt`` / ``.prototxt``, the
    text alone (with the parameters inside when ``include_params``)."""
    ext = extension if hasattr(filename, "write") else os.path.splitext(filename)[1]
    if parameter_format != ".protobuf":
        raise NotImplementedError("save: parameters are written as .protobuf only")
    if ext == ".nnp":
        root, used = create_proto(contents, False, variable_batch_size)
        if parameters is not None:
            used = OrderedDict(parameters)
        blob = OrderedDict((n, (v.d, bool(v.need_grad))) for n, v in used.items())
        buf = io.BytesIO()
        with zipfile.ZipFile(buf, "w") as z:
            z.writestr("nnp_version.txt", "0.1\n")
            z.writestr("network.nntxt", nnp_format.format_text(root))
            z.writestr("parameter.protobuf", nnp_format.encode_parameters(blob))
        data = buf.getvalue()
    elif ext in (".nntxt", ".prototxt"):
        root, _ = create_proto(contents, include_params, variable_batch_size)
        data = nnp_format.format_text(root).encode("utf-8")
    else:
        raise NotImplementedError("save: format %r is not supported (.nnp, .nntxt, .prototxt)" % ext)
    if hasattr(filename, "write"):
        filename.write(data)
    else:
        with open(filename, "wb") as fh:
            fh.write(data)
