"""The two encodings an NNP archive uses, for the subset of nnabla.proto the quantized graphs need
(src/nbla/proto/nnabla.proto.tmpl:24-48,64-110,265-323):

* protobuf *text* format for the network definition (``*.nntxt`` / ``*.prototxt``): parsed into nested
  :class:`Message` objects without a schema (field names are kept as written, repeated fields as lists);
* protobuf *wire* format for the parameters (``parameter.protobuf``): ``NNablaProtoBuf.parameter`` (field 200), each a
  ``Parameter {variable_name = 1; Shape shape = 20 {repeated int64 dim = 1}; repeated float data = 100;
  bool need_grad = 101}``.

Writers for both are included so that graphs can be saved and the readers tested by round trips.
"""
import struct
from collections import OrderedDict

import numpy as np


class NnpFormatError(ValueError):
    pass


# ------------------------------------------------------------------------------------------------ text format

class Message(object):
    """Fields of one text-format message in file order; every field name maps to the list of its values."""

    def __init__(self):
        self.fields = OrderedDict()

    def add(self, name, value):
        self.fields.setdefault(name, []).append(value)

    def all(self, name):
        return list(self.fields.get(name, ()))

    def get(self, name, default=None):
        v = self.fields.get(name)
        return v[-1] if v else default

    def has(self, name):
        return name in self.fields

    def __repr__(self):
        return "Message(%s)" % ", ".join("%s=%r" % kv for kv in self.fields.items())


class _Name(str):
    """A bare identifier value (enum name, true/false, inf/nan) as opposed to a quoted string."""


_ESCAPES = {"n": "\n", "t": "\t", "r": "\r", "\\": "\\", '"': '"', "'": "'", "0": "\0"}


def _tokens(text):
    i, n = 0, len(text)
    while i < n:
        c = text[i]
        if c.isspace() or c in ",;":
            i += 1
        elif c == "#":
            while i < n and text[i] != "\n":
                i += 1
        elif c in "{}:<>[]":
            yield c, c
            i += 1
        elif c in "\"'":
            j, out = i + 1, []
            while True:
                if j >= n:
                    raise NnpFormatError("unterminated string starting at offset %d" % i)
                if text[j] == "\\" and j + 1 < n:
                    out.append(_ESCAPES.get(text[j + 1], text[j + 1]))
                    j += 2
                elif text[j] == c:
                    break
                else:
                    out.append(text[j])
                    j += 1
            yield "str", "".join(out)
            i = j + 1
        else:
            j = i
            while j < n and not text[j].isspace() and text[j] not in "{}:<>[],;#\"'":
                j += 1
            yield "atom", text[i:j]
            i = j


def _atom(tok):
    low = tok.lower()
    if low == "true":
        return True
    if low == "false":
        return False
    try:
        return int(tok, 0)
    except ValueError:
        pass
    try:
        return float(tok[:-1] if low.endswith("f") and low not in ("inf", "-inf") else tok)
    except ValueError:
        return _Name(tok)


def parse_text(text):
    """Parse protobuf text format into a :class:`Message` tree."""
    toks = list(_tokens(text))
    pos = [0]

    def message(closer):
        m = Message()
        while True:
            if pos[0] >= len(toks):
                if closer is None:
                    return m
                raise NnpFormatError("missing %r at the end of the text" % closer)
            kind, val = toks[pos[0]]
            if closer is not None and val == closer and kind == closer:
                pos[0] += 1
                return m
            if kind != "atom":
                raise NnpFormatError("expected a field name, found %r" % (val,))
            name = val
            pos[0] += 1
            if pos[0] < len(toks) and toks[pos[0]][0] == ":":
                pos[0] += 1
            if pos[0] >= len(toks):
                raise NnpFormatError("field %r has no value" % name)
            kind, val = toks[pos[0]]
            pos[0] += 1
            if kind == "{":
                m.add(name, message("}"))
            elif kind == "<":
                m.add(name, message(">"))
            elif kind == "[":
                while True:
                    kind, val = toks[pos[0]]
                    pos[0] += 1
                    if kind == "]":
                        break
                    m.add(name, val if kind == "str" else _atom(val))
            elif kind == "str":
                # adjacent string literals concatenate
                while pos[0] < len(toks) and toks[pos[0]][0] == "str":
                    val += toks[pos[0]][1]
                    pos[0] += 1
                m.add(name, val)
            elif kind == "atom":
                m.add(name, _atom(val))
            else:
                raise NnpFormatError("field %r: unexpected %r" % (name, val))

    return message(None)


def _text_value(v):
    if isinstance(v, bool):
        return "true" if v else "false"
    if isinstance(v, _Name):
        return str(v)
    if isinstance(v, str):
        return '"%s"' % v.replace("\\", "\\\\").replace('"', '\\"').replace("\n", "\\n")
    if isinstance(v, float):
        return repr(float(v))
    return str(v)


def format_text(msg, indent=0):
    """Inverse of :func:`parse_text`."""
    pad, out = "  " * indent, []
    for name, values in msg.fields.items():
        for v in values:
            if isinstance(v, Message):
                out.append("%s%s {\n%s%s}\n" % (pad, name, format_text(v, indent + 1), pad))
            else:
                out.append("%s%s: %s\n" % (pad, name, _text_value(v)))
    return "".join(out)


# ------------------------------------------------------------------------------------------------ wire format

def _varint(buf, pos):
    shift = result = 0
    while True:
        if pos >= len(buf):
            raise NnpFormatError("truncated varint")
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7
        if shift > 63:
            raise NnpFormatError("varint longer than 64 bits")


def _fields(buf):
    """Yield (field number, wire type, value) of one message; length-delimited values come as memoryviews."""
    pos, view = 0, memoryview(buf)
    while pos < len(view):
        key, pos = _varint(view, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(view, pos)
        elif wt == 1:
            val, pos = bytes(view[pos:pos + 8]), pos + 8
        elif wt == 2:
            ln, pos = _varint(view, pos)
            if pos + ln > len(view):
                raise NnpFormatError("length-delimited field %d runs past the end of its message" % num)
            val, pos = view[pos:pos + ln], pos + ln
        elif wt == 5:
            val, pos = bytes(view[pos:pos + 4]), pos + 4
        else:
            raise NnpFormatError("unsupported wire type %d (field %d)" % (wt, num))
        yield num, wt, val


def _signed64(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _decode_shape(buf):
    dims = []
    for num, wt, val in _fields(buf):
        if num != 1:
            continue
        if wt == 0:
            dims.append(_signed64(val))
        elif wt == 2:  # packed
            pos = 0
            while pos < len(val):
                d, pos = _varint(val, pos)
                dims.append(_signed64(d))
    return tuple(dims)


def _decode_parameter(buf):
    name, shape, need_grad = "", (), False
    chunks = []
    for num, wt, val in _fields(buf):
        if num == 1 and wt == 2:
            name = bytes(val).decode("utf-8")
        elif num == 20 and wt == 2:
            shape = _decode_shape(val)
        elif num == 100 and wt == 2:  # packed floats
            if len(val) % 4:
                raise NnpFormatError("parameter %r: packed float data of %d bytes" % (name, len(val)))
            chunks.append(np.frombuffer(val, dtype="<f4"))
        elif num == 100 and wt == 5:
            chunks.append(np.frombuffer(val, dtype="<f4"))
        elif num == 101 and wt == 0:
            need_grad = bool(val)
    data = np.concatenate(chunks) if chunks else np.zeros(0, np.float32)
    size = int(np.prod(shape, dtype=np.int64)) if shape else data.size
    if data.size != size:
        raise NnpFormatError("parameter %r: %d values for shape %s" % (name, data.size, shape))
    return name, data.astype(np.float32).reshape(shape if shape else data.shape), need_grad


def decode_parameters(buf):
    """``parameter.protobuf`` -> OrderedDict name -> (float32 array, need_grad)."""
    out = OrderedDict()
    for num, wt, val in _fields(buf):
        if num == 200 and wt == 2:
            name, data, need_grad = _decode_parameter(val)
            out[name] = (data, need_grad)
    return out


def _enc_varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _enc_field(num, payload):
    return _enc_varint((num << 3) | 2) + _enc_varint(len(payload)) + payload


def encode_parameters(params):
    """Mapping name -> array or (array, need_grad) -> bytes of an NNablaProtoBuf holding only parameters."""
    out = []
    for name, v in params.items():
        data, need_grad = v if isinstance(v, tuple) else (v, True)
        data = np.asarray(data)
        shape = b"".join(_enc_varint((1 << 3) | 0) + _enc_varint(int(d)) for d in data.shape)
        body = _enc_field(1, name.encode("utf-8")) + _enc_field(20, shape)
        body += _enc_field(100, np.ascontiguousarray(data, dtype="<f4").tobytes())
        body += _enc_varint((101 << 3) | 0) + _enc_varint(1 if need_grad else 0)
        out.append(_enc_field(200, body))
    return b"".join(out)


def pack_float(v):
    return struct.pack("<f", v)


# ------------------------------------------------------------------- wire format of the network definition
# The messages of nnabla.proto.tmpl a network definition uses, as {field name: (number, type)}; a type is a scalar kind
# ('string', 'int64', 'bool', 'float'), the name of another message of this table, or ('repeated', type).
# Function.<type>_param has the number 1001 + the position of the function in functions.yaml, and the fields of a
# <Type>Parameter message are the function's arguments in the order of functions.yaml, numbered from 1
# (nnabla.proto.tmpl:300-323); the positions below are those of build-tools/code_generator/functions.yaml.
_CONV = [("base_axis", "int64"), ("pad", "Shape"), ("stride", "Shape"), ("dilation", "Shape"), ("group", "int64")]
_FUNCTION_PARAMS = OrderedDict([
    # snake name: (position in functions.yaml, arguments)
    ("affine", (0, [("base_axis", "int64")])),
    ("convolution", (4, _CONV + [("channel_last", "bool")])),
    ("relu", (21, [("inplace", "bool")])),
    ("add2", (64, [("inplace", "bool")])),
    ("sub2", (67, [("inplace", "bool")])),
    ("mul2", (68, [("inplace", "bool")])),
    ("div2", (70, [("inplace", "bool")])),
    ("pow2", (71, [("inplace", "bool")])),
    ("concatenate", (132, [("axis", "int64")])),
    ("binary_connect_affine", (201, [("base_axis", "int64"), ("quantize_zero_to", "float")])),
    ("binary_connect_convolution", (202, _CONV + [("quantize_zero_to", "float")])),
    ("binary_weight_affine", (203, [("base_axis", "int64"), ("quantize_zero_to", "float")])),
    ("binary_weight_convolution", (204, _CONV + [("quantize_zero_to", "float")])),
    ("inq_affine", (205, [("base_axis", "int64"), ("num_bits", "int64"), ("inq_iterations", ("repeated", "int64")),
                          ("selection_algorithm", "string"), ("seed", "int64")])),
    ("inq_convolution", (206, _CONV + [("num_bits", "int64"), ("inq_iterations", ("repeated", "int64")),
                                       ("selection_algorithm", "string"), ("seed", "int64")])),
    ("fixed_point_quantize", (207, [("sign", "bool"), ("n", "int64"), ("delta", "float"),
                                    ("ste_fine_grained", "bool")])),
    ("min_max_quantize", (208, [("decay", "float"), ("x_min_max", "bool"), ("ema", "bool"),
                                ("ste_fine_grained", "bool"), ("eps", "float")])),
    ("pow2_quantize", (209, [("sign", "bool"), ("with_zero", "bool"), ("n", "int64"), ("m", "int64"),
                             ("ste_fine_grained", "bool")])),
    ("prune", (210, [("rate", "float")])),
    ("quantize_linear", (211, [("round_mode", "string"), ("narrow_range", "bool"), ("dtype", "int64")])),
])


def _build_schema():
    rep = lambda t: ("repeated", t)
    s = {
        "Shape": {"dim": (1, rep("int64"))},
        "Context": {"backends": (1, rep("string")), "array_class": (2, "string"), "device_id": (3, "string"),
                    "backend": (4, "string"), "compute_backend": (5, "string")},
        "GlobalConfig": {"default_context": (1, "Context")},
        "NNablaProtoBuf": {"version": (1, "string"), "global_config": (2, "GlobalConfig"),
                           "network": (100, rep("Network")), "parameter": (200, rep("Parameter")),
                           "executor": (600, rep("Executor"))},
        "Network": {"name": (1, "string"), "batch_size": (10, "int64"), "repeat_info": (11, rep("RepeatInfo")),
                    "variable": (100, rep("Variable")), "function": (200, rep("Function"))},
        "RepeatInfo": {"id": (1, "string"), "times": (2, "int64")},
        "RepeatParameter": {"repeat_id": (1, "string"), "times": (2, "int64")},
        "RecurrentParameter": {"repeat_id": (1, "string"), "length": (2, "int64"), "axis": (3, "int64")},
        "Variable": {"name": (1, "string"), "type": (2, "string"), "repeat_id": (3, rep("string")),
                     "shape": (20, "Shape"), "initializer": (100, "Initializer")},
        "Initializer": {"type": (2, "string"), "multiplier": (10, "float")},
        "Parameter": {"variable_name": (1, "string"), "shape": (20, "Shape"), "data": (100, rep("float")),
                      "need_grad": (101, "bool")},
        "Executor": {"name": (1, "string"), "network_name": (10, "string"), "num_evaluations": (20, "int64"),
                     "repeat_evaluation_type": (21, "string"), "need_back_propagation": (30, "bool"),
                     "data_variable": (50, rep("DataVariable")), "generator_variable": (60, rep("GeneratorVariable")),
                     "loss_variable": (70, rep("LossVariable")), "output_variable": (80, rep("OutputVariable")),
                     "parameter_variable": (90, rep("ParameterVariable")), "no_image_normalization": (101, "bool")},
        "DataVariable": {"variable_name": (1, "string"), "data_name": (3, "string")},
        "GeneratorVariable": {"variable_name": (1, "string"), "type": (2, "string"), "multiplier": (3, "float")},
        "LossVariable": {"variable_name": (1, "string")},
        "OutputVariable": {"variable_name": (1, "string"), "type": (2, "string"), "data_name": (3, "string")},
        "ParameterVariable": {"variable_name": (1, "string"), "learning_rate_multiplier": (2, "float")},
        "Function": {"name": (1, "string"), "type": (2, "string"), "repeat_id": (3, rep("string")),
                     "context": (10, "Context"), "input": (20, rep("string")), "output": (30, rep("string")),
                     "repeat_param": (100, "RepeatParameter"), "recurrent_param": (101, "RecurrentParameter")},
    }
    for snake, (position, args) in _FUNCTION_PARAMS.items():
        msg = "".join(p.capitalize() for p in snake.split("_")) + "Parameter"
        s["Function"][snake + "_param"] = (1001 + position, msg)
        s[msg] = {name: (i + 1, kind) for i, (name, kind) in enumerate(args)}
    return s


WIRE_SCHEMA = _build_schema()
_SCALAR_WIRE = {"string": 2, "int64": 0, "bool": 0, "float": 5}


def _decode_scalar(kind, wt, val, where):
    if kind == "string" and wt == 2:
        return bytes(val).decode("utf-8")
    if kind == "int64" and wt == 0:
        return _signed64(val)
    if kind == "bool" and wt == 0:
        return bool(val)
    if kind == "float" and wt == 5:
        return struct.unpack("<f", val)[0]
    raise NnpFormatError("%s: wire type %d does not fit a %s" % (where, wt, kind))


def decode_message(buf, message="NNablaProtoBuf", skip=()):
    """Wire-format bytes of a message of WIRE_SCHEMA -> the :class:`Message` tree the text parser would give (same
    field names; fields the schema does not list, e.g. the parameter messages of functions outside this path, are
    left out, and so are the fields named in ``skip``)."""
    fields = WIRE_SCHEMA[message]
    by_number = {num: (name, kind) for name, (num, kind) in fields.items()}
    out = Message()
    for num, wt, val in _fields(buf):
        if num not in by_number:
            continue
        name, kind = by_number[num]
        if name in skip:
            continue
        where = "%s.%s" % (message, name)
        repeated = isinstance(kind, tuple)
        if repeated:
            kind = kind[1]
        if kind in WIRE_SCHEMA:
            if wt != 2:
                raise NnpFormatError("%s: wire type %d for a message" % (where, wt))
            out.add(name, decode_message(val, kind))
        elif repeated and wt == 2 and kind != "string":      # packed
            if kind == "float":
                if len(val) % 4:
                    raise NnpFormatError("%s: packed floats of %d bytes" % (where, len(val)))
                for f in np.frombuffer(val, dtype="<f4"):
                    out.add(name, float(f))
            else:
                pos = 0
                while pos < len(val):
                    v, pos = _varint(val, pos)
                    out.add(name, bool(v) if kind == "bool" else _signed64(v))
        else:
            out.add(name, _decode_scalar(kind, wt, val, where))
    return out


def encode_message(msg, message="NNablaProtoBuf"):
    """Inverse of :func:`decode_message` (repeated numbers are written packed, as proto3 writers do)."""
    fields = WIRE_SCHEMA[message]
    out = []
    for name, values in msg.fields.items():
        if name not in fields:
            raise NnpFormatError("%s has no field %r in the wire schema" % (message, name))
        num, kind = fields[name]
        repeated = isinstance(kind, tuple)
        if repeated:
            kind = kind[1]
        if kind in WIRE_SCHEMA:
            for v in values:
                out.append(_enc_field(num, encode_message(v, kind)))
        elif repeated and kind != "string":
            if kind == "float":
                body = np.asarray([float(v) for v in values], dtype="<f4").tobytes()
            else:
                body = b"".join(_enc_varint(int(v)) for v in values)
            out.append(_enc_field(num, body))
        else:
            for v in values:
                if kind == "string":
                    out.append(_enc_field(num, str(v).encode("utf-8")))
                elif kind == "float":
                    out.append(_enc_varint((num << 3) | 5) + struct.pack("<f", float(v)))
                else:
                    out.append(_enc_varint((num << 3) | 0) + _enc_varint(int(v)))
    return b"".join(out)
