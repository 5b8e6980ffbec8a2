"""Writing graphs as NNP files and reading them back (host side: graph construction and shape inference only)."""
import io
import zipfile

import numpy as np
import pytest

import nnabla_amd as nn
import nnabla_amd.functions as F
import nnabla_amd.parametric_functions as PF
from nnabla_amd.ext_utils import get_extension_context
from nnabla_amd.utils import nnp_format, qnn
from nnabla_amd.utils.nnp_graph import NnpLoader
from nnabla_amd.utils.save import save


@pytest.fixture(autouse=True)
def hip_scope():
    nn.clear_parameters()
    with nn.context_scope(get_extension_context('hip')):
        yield
    nn.clear_parameters()


def graph_info(v):
    out = []
    v.visit(lambda f: out.append((f.info.type_name, dict(f.info.args), [tuple(i.shape) for i in f.inputs],
                                  [tuple(o.shape) for o in f.outputs])))
    return out


def every_function_net(x):
    """One function of every storable type, each with non-default arguments."""
    rng = np.random.RandomState(0)

    def p(name, shape, need_grad=True):
        data = rng.randn(*shape).astype(np.float32)
        if name.endswith('/I'):
            data = (data > 0).astype(np.float32)      # INQ indicators: the loader stores them as integers
        return nn.parameter.get_parameter_or_create(name, shape, data, need_grad)

    h = F.convolution(x, p('conv/W', (4, 3, 3, 3)), p('conv/b', (4,)), pad=(1, 1), stride=(1, 1), dilation=(1, 1))
    h = F.relu(h)
    h = F.div2(F.mul2(h, F.relu(h)), F.sub2(h, F.add2(h, h)))
    h = F.fixed_point_quantize(h, False, 6, 0.25, ste_fine_grained=False)
    h = F.pow2_quantize(h, True, False, 5, 2)
    h = F.min_max_quantize(h, p('mmq/qr_min', (1, 1, 1, 1), False), p('mmq/qr_max', (1, 1, 1, 1), False),
                           p('mmq/ql_min', (1, 1, 1, 1), False), p('mmq/ql_max', (1, 1, 1, 1), False), decay=0.9,
                           x_min_max=True, ema=True, eps=0.02)
    h = F.binary_weight_convolution(h, p('bwc/W', (4, 4, 3, 3)), p('bwc/Wb', (4, 4, 3, 3), False),
                                    p('bwc/alpha', (4,), False), None, pad=(1, 1), quantize_zero_to=-1.0)
    h = F.binary_connect_convolution(h, p('bcc/W', (4, 4, 3, 3)), p('bcc/Wb', (4, 4, 3, 3), False), p('bcc/b', (4,)),
                                     stride=(2, 2))
    h = F.inq_convolution(h, p('inqc/W', (4, 4, 1, 1)), p('inqc/I', (4, 4, 1, 1), False), None, num_bits=3,
                          inq_iterations=(10, 20), selection_algorithm='random', seed=5)
    h = F.prune(h, 0.25)
    h = F.quantize_linear(h, p('ql/s', (1, 1, 1, 1), False), p('ql/z', (1, 1, 1, 1), False), 'HALF_TO_EVEN', True,
                          np.uint8)
    h = F.dequantize_linear(h, p('ql/s', (1, 1, 1, 1), False), p('ql/z', (1, 1, 1, 1), False))
    h = F.affine(h, p('a/W', (16, 12)), p('a/b', (12,)))
    h = F.binary_weight_affine(h, p('bwa/W', (12, 10)), p('bwa/Wb', (12, 10), False), p('bwa/alpha', (10,), False),
                               p('bwa/b', (10,)), quantize_zero_to=-1.0)
    h = F.binary_connect_affine(h, p('bca/W', (10, 9)), p('bca/Wb', (10, 9), False))
    return F.inq_affine(h, p('inqa/W', (9, 7)), p('inqa/I', (9, 7), False), p('inqa/b', (7,)), num_bits=5,
                        inq_iterations=(3,), selection_algorithm='largest_abs', seed=-1)


def contents_of(x, y, batch):
    return {'networks': [{'name': 'net', 'batch_size': batch, 'outputs': {'y': y}, 'names': {'x': x}}],
            'executors': [{'name': 'runtime', 'network': 'net', 'data': ['x'], 'output': ['y']}]}


def test_every_function_round_trip():
    x = nn.Variable((6, 3, 6, 6))
    y = every_function_net(x)
    want = graph_info(y)
    stored = {k: v.d.copy() for k, v in nn.get_parameters(grad_only=False).items()}
    grads = {k: v.need_grad for k, v in nn.get_parameters(grad_only=False).items()}
    buf = io.BytesIO()
    save(buf, contents_of(x, y, 6), extension='.nnp')
    nn.clear_parameters()

    with zipfile.ZipFile(io.BytesIO(buf.getvalue())) as z:
        assert sorted(z.namelist()) == ['network.nntxt', 'nnp_version.txt', 'parameter.protobuf']
        text = z.read('network.nntxt').decode()
    root = nnp_format.parse_text(text)
    net_msg = root.get('network')
    dims = {str(v.get('name')): [int(d) for d in v.get('shape').all('dim')] for v in net_msg.all('variable')}
    assert dims['x'] == [-1, 3, 6, 6] and dims['y'] == [-1, 7] and dims['conv/W'] == [4, 3, 3, 3]
    assert [str(v.get('type')) for v in net_msg.all('variable') if str(v.get('name')) in ('x', 'y', 'a/W')] == \
        ['Buffer', 'Parameter', 'Buffer']
    exe = root.get('executor')
    assert str(exe.get('network_name')) == 'net'
    assert [str(d.get('variable_name')) for d in exe.all('data_variable')] == ['x']
    assert [str(d.get('variable_name')) for d in exe.all('output_variable')] == ['y']
    assert sorted(str(d.get('variable_name')) for d in exe.all('parameter_variable')) == sorted(stored)

    loader = NnpLoader(io.BytesIO(buf.getvalue()), extension='.nnp')
    for batch in (6, 2):
        net = loader.get_network('net', batch_size=batch)
        got = graph_info(net.outputs['y'])
        assert [g[:2] for g in got] == [w[:2] for w in want]          # types and every argument
        if batch == 6:
            assert got == want
        assert list(net.inputs) == ['x'] and net.inputs['x'].shape == (batch, 3, 6, 6)
        assert net.outputs['y'].shape == (batch, 7)
    params = loader.get_parameters()
    assert sorted(params) == sorted(stored)
    for k, v in stored.items():
        assert np.array_equal(params[k].d, v) and params[k].need_grad == grads[k], k
    ex = loader.get_executor('runtime')
    assert list(ex.data_variables) == ['x'] and list(ex.output_variables) == ['y']


def test_text_formats_and_parameters_inside():
    x = nn.Variable((2, 5))
    y = F.relu(PF.affine(x, 3, name='fc'))
    W = nn.get_parameter('fc/affine/W').d
    for ext in ('.nntxt', '.prototxt'):
        buf = io.BytesIO()
        save(buf, contents_of(x, y, 2), include_params=True, variable_batch_size=False, extension=ext)
        root = nnp_format.parse_text(buf.getvalue().decode())
        assert [int(d) for d in root.get('network').all('variable')[0].get('shape').all('dim')] == [2, 5]
        loader = NnpLoader(io.BytesIO(buf.getvalue()), extension=ext)
        assert np.array_equal(loader.get_parameters()['fc/affine/W'].d, W)
        assert loader.get_parameters()['fc/affine/W'].need_grad
        assert [f.info.type_name for f in [loader.get_network('net').outputs['y'].parent]] == ['ReLU']
    buf = io.BytesIO()
    save(buf, contents_of(x, y, 2), extension='.nntxt')
    assert 'parameter {' not in buf.getvalue().decode()


def test_converted_graphs_keep_their_names(tmp_path):
    """Graph converters hand a function unlinked views of the graph inputs and of the first layer's parameters:
    they are stored under the names of the variables they view."""
    import nnabla_amd.experimental.graph_converters as GC
    x = nn.Variable((2, 5))
    y = PF.affine(F.relu(PF.affine(x, 4, name='fc1')), 3, name='fc2')
    y2 = GC.GraphConverter([GC.FunctionModifier()]).convert(y)
    path = str(tmp_path / 'net.nnp')
    save(path, contents_of(x, y2, 2))
    net = NnpLoader(path).get_network('net')
    assert list(net.inputs) == ['x']
    assert [n for n in net.variables if '/' in n] == ['fc1/affine/W', 'fc1/affine/b', 'fc2/affine/W', 'fc2/affine/b']


def test_errors():
    x = nn.Variable((2, 5))
    y = PF.affine(x, 3, name='fc')
    with pytest.raises(ValueError, match="MaxMaxRecorder"):
        save(io.BytesIO(), contents_of(x, qnn.max_max_recorder(y, nn.Variable((1, 1))), 2))
    c = contents_of(x, y, 2)
    c['executors'][0]['data'] = ['nope']
    with pytest.raises(ValueError, match="nope"):
        save(io.BytesIO(), c)
    c = contents_of(x, y, 2)
    c['executors'][0]['network'] = 'other'
    with pytest.raises(ValueError, match="other"):
        save(io.BytesIO(), c)
    c = contents_of(x, y, 2)
    c['optimizers'] = [{'name': 'o'}]
    with pytest.raises(NotImplementedError):
        save(io.BytesIO(), c)
    with pytest.raises(NotImplementedError):
        save(io.BytesIO(), contents_of(x, y, 2), extension='.protobuf')
    with pytest.raises(NotImplementedError):
        save(io.BytesIO(), contents_of(x, y, 2), parameter_format='.h5')
    # an input nobody named gets a generated name; one that collides with a given name is refused
    buf = io.BytesIO()
    save(buf, {'networks': [{'name': 'n', 'batch_size': 2, 'outputs': {'y': y}}]}, extension='.nntxt')
    assert list(NnpLoader(io.BytesIO(buf.getvalue())).get_network('n').inputs) == ['Input_1']
    other = nn.Variable((2, 3))
    with pytest.raises(ValueError, match="named"):
        save(io.BytesIO(), {'networks': [{'name': 'n', 'batch_size': 2, 'outputs': {'y': y, 'z': F.relu(other)},
                                          'names': {'Input_1': other}}]})
