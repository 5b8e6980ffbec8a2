"""NNP file handling on the CPU: the text and wire codecs cross-checked against google.protobuf (descriptors built
at run time from the field numbers of src/nbla/proto/nnabla.proto.tmpl:24-48,64-110), archive round trips, graph
construction (shapes, inputs/outputs, batch size) and the error paths.  Nothing here runs a kernel."""
import io
import zipfile

import numpy as np
import pytest

import nnabla_amd as nn
from nnabla_amd.ext_utils import get_extension_context
from nnabla_amd.utils import nnp_format
from nnabla_amd.utils.nnp_graph import NnpError, NnpLoader, SUPPORTED_FUNCTIONS, save_nnp

NET = '''
# a two-layer quantized network
global_config { default_context { array_class: "HipCachedArray" device_id: "0" backends: "hip:float" } }
network {
  name: "net"
  batch_size: 4
  variable { name: "x" type: "Buffer" shape: { dim: -1 dim: 8 } }
  variable { name: "W" type: "Parameter" shape: { dim: 8 dim: 6 } initializer { type: "Normal" multiplier: 0.5 } }
  variable { name: "Wb" type: "Parameter" shape: { dim: 8 dim: 6 } initializer { type: "Constant" multiplier: 0 } }
  variable { name: "alpha" type: "Parameter" shape: { dim: 6 } }
  variable { name: "q" type: "Buffer" shape: { dim: -1 dim: 8 } }
  variable { name: "y" type: "Buffer" shape: { dim: -1 dim: 6 } }
  variable { name: "r" type: "Buffer" shape: { dim: -1 dim: 6 } }
  function {
    name: "Q" type: "FixedPointQuantize" input: "x" output: "q"
    fixed_point_quantize_param { sign: true n: 8 delta: 0.0625 ste_fine_grained: true }
  }
  function {
    name: "A" type: "BinaryWeightAffine" input: "q" input: "W" input: "Wb" input: "alpha" output: "y"
    binary_weight_affine_param { base_axis: 1 quantize_zero_to: 1.0 }
  }
  function { name: "R" type: "ReLU" input: "y" output: "r" relu_param { inplace: false } }
}
executor {
  name: "run" network_name: "net"
  data_variable { variable_name: "x" data_name: "input" }
  output_variable { variable_name: "r" data_name: "result" }
}
'''


@pytest.fixture()
def hip_ctx():
    with nn.context_scope(get_extension_context('hip', device_id='0')):
        yield


def _pb_classes():
    """Message classes for the parameter subset of nnabla.proto, built without protoc."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    fd = descriptor_pb2.FileDescriptorProto(name="nnabla_subset.proto", syntax="proto3")
    T = descriptor_pb2.FieldDescriptorProto
    shape = fd.message_type.add(name="Shape")
    shape.field.add(name="dim", number=1, type=T.TYPE_INT64, label=T.LABEL_REPEATED)
    par = fd.message_type.add(name="Parameter")
    par.field.add(name="variable_name", number=1, type=T.TYPE_STRING, label=T.LABEL_OPTIONAL)
    par.field.add(name="shape", number=20, type=T.TYPE_MESSAGE, type_name=".Shape", label=T.LABEL_OPTIONAL)
    par.field.add(name="data", number=100, type=T.TYPE_FLOAT, label=T.LABEL_REPEATED)
    par.field.add(name="need_grad", number=101, type=T.TYPE_BOOL, label=T.LABEL_OPTIONAL)
    root = fd.message_type.add(name="NNablaProtoBuf")
    root.field.add(name="version", number=1, type=T.TYPE_STRING, label=T.LABEL_OPTIONAL)
    root.field.add(name="parameter", number=200, type=T.TYPE_MESSAGE, type_name=".Parameter", label=T.LABEL_REPEATED)
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return message_factory.GetMessageClass(pool.FindMessageTypeByName("NNablaProtoBuf"))


def test_wire_decoder_reads_what_protobuf_writes():
    Root = _pb_classes()
    rng = np.random.RandomState(0)
    w = rng.randn(3, 4, 5).astype(np.float32)
    msg = Root(version="x")
    p = msg.parameter.add(variable_name="conv/W", need_grad=True)
    p.shape.dim.extend(w.shape)
    p.data.extend(w.ravel().tolist())
    p = msg.parameter.add(variable_name="scalar")            # need_grad false, shape (1,)
    p.shape.dim.append(1)
    p.data.append(-2.5)
    p = msg.parameter.add(variable_name="big_dim")
    p.shape.dim.extend([300, 1])                             # a dim that needs a two-byte varint
    p.data.extend(np.arange(300, dtype=np.float32).tolist())
    got = nnp_format.decode_parameters(msg.SerializeToString())
    assert list(got) == ["conv/W", "scalar", "big_dim"]
    assert np.array_equal(got["conv/W"][0], w) and got["conv/W"][1] is True
    assert got["scalar"][0].shape == (1,) and got["scalar"][0][0] == -2.5 and got["scalar"][1] is False
    assert got["big_dim"][0].shape == (300, 1) and got["big_dim"][0][299, 0] == 299


def test_protobuf_reads_what_the_wire_encoder_writes():
    Root = _pb_classes()
    rng = np.random.RandomState(1)
    params = {"a/W": rng.randn(7, 130).astype(np.float32), "a/b": (np.float32([1, 2, 3]), False)}
    msg = Root()
    msg.ParseFromString(nnp_format.encode_parameters(params))
    assert [p.variable_name for p in msg.parameter] == ["a/W", "a/b"]
    assert list(msg.parameter[0].shape.dim) == [7, 130] and msg.parameter[0].need_grad
    assert np.array_equal(np.float32(msg.parameter[0].data).reshape(7, 130), params["a/W"])
    assert list(msg.parameter[1].data) == [1, 2, 3] and not msg.parameter[1].need_grad
    # and the decoder inverts the encoder bit for bit, including NaN payloads and signed zeros
    odd = np.array([np.nan, -0.0, np.inf, 1e-45], np.float32)
    back = nnp_format.decode_parameters(nnp_format.encode_parameters({"o": odd}))["o"][0]
    assert np.array_equal(back.view(np.uint32), odd.view(np.uint32))


def test_wire_decoder_rejects_damaged_input():
    good = nnp_format.encode_parameters({"w": np.zeros((2, 2), np.float32)})
    with pytest.raises(nnp_format.NnpFormatError):
        nnp_format.decode_parameters(good[:-3])
    bad_count = nnp_format.encode_parameters({"w": np.zeros(3, np.float32)}).replace(b"\x08\x03", b"\x08\x04")
    with pytest.raises(nnp_format.NnpFormatError):
        nnp_format.decode_parameters(bad_count)


def test_text_parser_against_protobuf_text_format():
    """The same text parsed by google.protobuf (for the parameter subset) and by the schema-less parser."""
    from google.protobuf import text_format
    Root = _pb_classes()
    text = '''version: "1"  # trailing comment
    parameter { variable_name: "w\\"q" shape { dim: 2 dim: 2 } data: 1.5 data: -2e-3 data: 3 data: 16 need_grad: true }
    parameter < variable_name: 'single' shape: { dim: 1 } data: [4.0, 5.5] >'''
    ref = text_format.Parse(text, Root())
    got = nnp_format.parse_text(text)
    assert got.get("version") == ref.version
    ps = got.all("parameter")
    assert len(ps) == len(ref.parameter) == 2
    for mine, theirs in zip(ps, ref.parameter):
        assert mine.get("variable_name") == theirs.variable_name
        assert [int(d) for d in mine.get("shape").all("dim")] == list(theirs.shape.dim)
        assert np.array_equal(np.float32([float(v) for v in mine.all("data")]), np.float32(list(theirs.data)))
        assert bool(mine.get("need_grad", False)) == theirs.need_grad
    # writer -> parser round trip keeps structure and values
    again = nnp_format.parse_text(nnp_format.format_text(got))
    assert nnp_format.format_text(again) == nnp_format.format_text(got)
    with pytest.raises(nnp_format.NnpFormatError):
        nnp_format.parse_text('network { name: "x" ')
    with pytest.raises(nnp_format.NnpFormatError):
        nnp_format.parse_text('name: "unterminated')


def test_graph_from_archive(tmp_path, hip_ctx):
    W = (np.arange(48, dtype=np.float32).reshape(8, 6) - 20) / 7
    path = str(tmp_path / "net.nnp")
    save_nnp(path, NET, {"W": W, "alpha": (np.zeros(6, np.float32), False)})
    assert set(zipfile.ZipFile(path).namelist()) >= {"network.nntxt", "parameter.protobuf"}
    loader = NnpLoader(path)
    assert loader.get_network_names() == ["net"] and loader.get_executor_names() == ["run"]
    net = loader.get_network("net")
    assert list(net.inputs) == ["x"] and list(net.outputs) == ["r"]
    assert net.variables["x"].shape == (4, 8) and net.variables["r"].shape == (4, 6)
    assert np.array_equal(net.variables["W"].d, W) and net.variables["W"].need_grad
    assert not net.variables["alpha"].need_grad
    assert not net.variables["Wb"].d.any()                      # Constant initializer, multiplier 0
    assert [n.info["type"] for n in (net.variables[k].parent for k in ("q", "y", "r"))] == [
        "FixedPointQuantize", "BinaryWeightAffine", "ReLU"]
    assert net.variables["q"].parent.info["fargs"] == (0.0625,)
    # batch size override; parameters are shared between the graphs of one loader
    net2 = loader.get_network("net", batch_size=9)
    assert net2.variables["x"].shape == (9, 8) and net2.variables["W"] is net.variables["W"]
    exe = loader.get_executor("run", batch_size=2)
    assert list(exe.data_variables) == ["input"] and exe.data_variables["input"].shape == (2, 8)
    assert list(exe.output_variables) == ["result"] and exe.output_variables["result"].shape == (2, 6)
    # a bare nntxt through a file object; W then comes from its Normal initializer
    net3 = NnpLoader(io.BytesIO(NET.encode()), extension=".nntxt").get_network("net")
    assert net3.variables["W"].d.std() > 0.1


def test_graph_errors(hip_ctx):
    def load(text):
        return NnpLoader(io.BytesIO(text.encode()), extension=".nntxt")
    with pytest.raises(NnpError, match="not available"):
        load(NET.replace('type: "ReLU"', 'type: "Softmax"')).get_network("net")
    with pytest.raises(NnpError, match="declares"):
        load(NET.replace('name: "y" type: "Buffer" shape: { dim: -1 dim: 6 }',
                         'name: "y" type: "Buffer" shape: { dim: -1 dim: 7 }')).get_network("net")
    with pytest.raises(NnpError, match="undefined"):
        load(NET.replace('input: "y" output: "r"', 'input: "nope" output: "r"')).get_network("net")
    with pytest.raises(NnpError, match="no network"):
        load(NET).get_network("other")
    with pytest.raises(NnpError, match="at least 4 inputs"):
        load(NET.replace('input: "alpha" ', '')).get_network("net")
    buf = io.BytesIO()
    with zipfile.ZipFile(buf, "w") as z:
        z.writestr("network.nntxt", NET)
        z.writestr("parameter.h5", b"\x89HDF")
    with pytest.raises(NnpError, match="HDF5"):
        NnpLoader(io.BytesIO(buf.getvalue()), extension=".nnp")
    assert set(SUPPORTED_FUNCTIONS) >= {"FixedPointQuantize", "Pow2Quantize", "MinMaxQuantize", "BinaryWeightAffine",
                                        "BinaryConnectAffine", "BinaryWeightConvolution",
                                        "BinaryConnectConvolution", "INQAffine", "INQConvolution"}


def test_linear_quantizer_and_prune_builders(hip_ctx):
    text = '''network { name: "q" batch_size: 2
      variable { name: "x" type: "Buffer" shape: { dim: -1 dim: 3 dim: 4 } }
      variable { name: "s" type: "Parameter" shape: { dim: 1 dim: 3 dim: 1 } initializer { type: "Constant" multiplier: 0.5 } }
      variable { name: "z" type: "Parameter" shape: { dim: 1 dim: 1 dim: 1 } }
      function { name: "p" type: "Prune" input: "x" output: "xp" prune_param { rate: 0.25 } }
      function { name: "q" type: "QuantizeLinear" input: "xp" input: "s" input: "z" output: "xq"
                 quantize_linear_param { round_mode: "HALF_TO_EVEN" narrow_range: true dtype: 2 } }
      function { name: "d" type: "DequantizeLinear" input: "xq" input: "s" input: "z" output: "y" }
    }'''
    net = NnpLoader(io.BytesIO(text.encode()), extension=".nntxt").get_network("q")
    v = net.variables
    assert list(net.outputs) == ["y"] and v["y"].shape == (2, 3, 4)
    assert v["xp"].parent.info == {"type": "Prune", "iargs": (), "fargs": (0.25,), "sarg": None}
    assert v["xq"].parent.info == {"type": "QuantizeLinear", "iargs": (1, 2), "fargs": (), "sarg": "HALF_TO_EVEN"}
    assert v["y"].parent.info["type"] == "DequantizeLinear"


# ------------------------------------------------------------------------------- networks in binary protobuf
def _pb_network_classes():
    """google.protobuf message classes for every message of nnp_format.WIRE_SCHEMA, built without protoc."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    T = descriptor_pb2.FieldDescriptorProto
    kinds = {"string": T.TYPE_STRING, "int64": T.TYPE_INT64, "bool": T.TYPE_BOOL, "float": T.TYPE_FLOAT}
    fd = descriptor_pb2.FileDescriptorProto(name="nnabla_networks.proto", syntax="proto3")
    for mname, fields in nnp_format.WIRE_SCHEMA.items():
        m = fd.message_type.add(name=mname)
        for fname, (num, kind) in fields.items():
            label = T.LABEL_OPTIONAL
            if isinstance(kind, tuple):
                label, kind = T.LABEL_REPEATED, kind[1]
            if kind in kinds:
                m.field.add(name=fname, number=num, type=kinds[kind], label=label)
            else:
                m.field.add(name=fname, number=num, type=T.TYPE_MESSAGE, type_name="." + kind, label=label)
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return message_factory.GetMessageClass(pool.FindMessageTypeByName("NNablaProtoBuf"))


def _tree(msg):
    """A Message tree as nested plain data, floats at float32 precision."""
    out = []
    for name, values in msg.fields.items():
        for v in values:
            if isinstance(v, nnp_format.Message):
                out.append((name, _tree(v)))
            elif isinstance(v, float):
                out.append((name, float(np.float32(v))))
            else:
                out.append((name, str(v) if isinstance(v, str) else v))
    return out


def test_function_message_known_bytes():
    """Function { name = 1; type = 2; input = 20; output = 30; relu_param = 1001 + 21 } with
    ReLUParameter { inplace = 1 }: the bytes written out by hand (nnabla.proto.tmpl:291-323; ReLU is the 22nd
    function of functions.yaml)."""
    want = (b"\x0a\x01f" b"\x12\x04ReLU" b"\xa2\x01\x01x" b"\xf2\x01\x01y"
            b"\xf2\x3f\x02\x08\x01")        # key (1022 << 3 | 2) = 8178 = f2 3f, length 2, inplace = true
    f = nnp_format.parse_text('name: "f" type: "ReLU" input: "x" output: "y" relu_param { inplace: true }')
    assert nnp_format.encode_message(f, "Function") == want
    back = nnp_format.decode_message(want, "Function")
    assert _tree(back) == _tree(f)
    # the field numbers of the quantization functions: positions 201..211 of functions.yaml
    nums = {k: v[0] for k, v in nnp_format.WIRE_SCHEMA["Function"].items() if k.endswith("_param")}
    assert nums["binary_connect_affine_param"] == 1202 and nums["quantize_linear_param"] == 1212
    assert nums["fixed_point_quantize_param"] == 1208 and nums["affine_param"] == 1001
    assert nums["add2_param"] == 1065 and nums["concatenate_param"] == 1133 and nums["convolution_param"] == 1005


def test_binary_network_round_trip_and_against_protobuf():
    root = nnp_format.parse_text(NET)
    wire = nnp_format.encode_message(root)
    assert _tree(nnp_format.decode_message(wire)) == _tree(root)
    Root = _pb_network_classes()
    pb = Root()
    pb.ParseFromString(wire)                      # google.protobuf reads what the encoder writes
    net = pb.network[0]
    assert net.name == "net" and net.batch_size == 4 and [v.name for v in net.variable][:2] == ["x", "W"]
    assert list(net.variable[0].shape.dim) == [-1, 8]
    f = net.function[0]
    assert f.type == "FixedPointQuantize" and list(f.input) == ["x"] and list(f.output) == ["q"]
    assert f.fixed_point_quantize_param.n == 8 and f.fixed_point_quantize_param.delta == 0.0625
    assert f.fixed_point_quantize_param.sign is True
    assert net.function[1].binary_weight_affine_param.base_axis == 1
    assert pb.executor[0].output_variable[0].variable_name == "r"
    assert abs(net.variable[1].initializer.multiplier - 0.5) < 1e-7
    # and the decoder reads what google.protobuf writes (packed repeated fields, default values left out)
    again = nnp_format.decode_message(pb.SerializeToString())
    a, b = _tree(again), _tree(root)
    # proto3 writers omit zeros and false, and write the fields in the order of their numbers
    drop = lambda t: sorted([(k, drop(v) if isinstance(v, list) else v) for k, v in t
                             if not (v is False or v == 0 or v == 0.0) or isinstance(v, list)], key=lambda kv: kv[0])
    assert drop(a) == drop(b)


def test_graph_from_binary_protobuf(tmp_path, hip_ctx):
    """An archive whose network definition is binary (load.py:492-494): the same graph as from the text."""
    rng = np.random.RandomState(1)
    params = {"W": rng.randn(8, 6).astype(np.float32), "alpha": np.ones(6, np.float32)}
    root = nnp_format.parse_text(NET)
    path = str(tmp_path / "binary.nnp")
    with zipfile.ZipFile(path, "w") as z:
        z.writestr("nnp_version.txt", "0.1\n")
        z.writestr("network.protobuf", nnp_format.encode_message(root))
        z.writestr("parameter.protobuf", nnp_format.encode_parameters(params))
    text_path = str(tmp_path / "text.nnp")
    save_nnp(text_path, NET, params)
    for p in (path, text_path):
        L = NnpLoader(p)
        assert L.get_network_names() == ["net"] and L.get_executor_names() == ["run"]
        net = L.get_network("net", batch_size=3)
        assert net.variables["r"].shape == (3, 6) and list(net.inputs) == ["x"] and list(net.outputs) == ["r"]
        assert np.array_equal(L.get_parameters()["W"].d, params["W"])
    # one .protobuf holding networks and parameters together
    both = nnp_format.encode_message(root) + nnp_format.encode_parameters(params)
    single = str(tmp_path / "all.protobuf")
    with open(single, "wb") as fh:
        fh.write(both)
    L = NnpLoader(single)
    assert L.get_network_names() == ["net"] and set(L.get_parameters()) >= {"W", "alpha"}
    assert L.get_network("net").variables["y"].shape == (4, 6)
