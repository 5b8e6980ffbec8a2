"""Host-side tests of the quantization-aware-training graph rewrites: graph bookkeeping of the front-end, the
converter driver, both quantization modifiers, the scale arithmetic and the scheduler.  Graph construction and shape
inference run without a GPU; nothing here executes a function.

The structure checks follow python/test/utils/test_graph_converters/test_quantize.py: the converted graph is compared
function by function (type names, input and output shapes, in forward order) with a graph written out by hand."""
import numpy as np
import pytest

import nnabla_amd as nn
import nnabla_amd.experimental.graph_converters as GC
import nnabla_amd.functions as F
import nnabla_amd.parametric_functions as PF
import oracle
from nnabla_amd.ext_utils import get_extension_context
from nnabla_amd.utils import qnn
from nnabla_amd.utils.qnn import FunctionsRankRecorder, QATConfig, QATScheduler, QNNState


@pytest.fixture(autouse=True)
def hip_scope():
    nn.clear_parameters()
    with nn.context_scope(get_extension_context('hip')):
        yield
    nn.clear_parameters()


def graph_info(v):
    out = []
    v.visit(lambda f: out.append((f.info.type_name, [tuple(i.shape) for i in f.inputs],
                                  [tuple(o.shape) for o in f.outputs])))
    return out


def names(v):
    return [n for n, _, _ in graph_info(v)]


def small_net(x):
    h = F.relu(PF.convolution(x, 4, (3, 3), name='c1'))
    h = F.relu(PF.convolution(h, 4, (3, 3), name='c2'))
    h = F.relu(PF.affine(h, 10, name='f1'))
    return PF.affine(h, 5, name='f2')


def params_of(scope):
    with nn.parameter_scope(scope):
        p = nn.get_parameters(grad_only=False)
    return p


# ------------------------------------------------------------------------------------------------ graph bookkeeping
def test_visit_order_references_and_rank():
    x = nn.Variable((4, 8))
    w, b = nn.Variable((8, 5)), nn.Variable((5,))
    h = F.affine(x, w, b)
    r = F.relu(h)
    end = F.sink(r, h)
    seen = []
    end.visit(lambda f: seen.append((f.info.type_name, f.rank)))
    assert seen == [('Affine', 0), ('ReLU', 1), ('Sink', 2)]
    assert end.shape == () and (x.rank, h.rank, r.rank, end.rank) == (0, 1, 2, 3)
    assert [f.info.type_name for f in h.function_references] == ['ReLU', 'Sink']
    assert [f.info.type_name for f in w.function_references] == ['Affine']
    assert h.parent.info.args == {'base_axis': 1}
    del end
    import gc
    gc.collect()
    assert [f.info.type_name for f in h.function_references] == ['ReLU']      # only live functions are listed


def test_function_clone_keeps_arguments():
    x = nn.Variable((2, 3, 8, 8))
    y = PF.convolution(x, 4, (3, 3), pad=(1, 1), stride=(2, 2), name='c')
    g = y.parent.function.clone()
    assert g.info == y.parent.info and g.info.args == y.parent.info.args
    assert g.info.args['pad'] == (1, 1) and g.info.args['stride'] == (2, 2)
    w, b = y.parent.inputs[1:]
    assert g(x, w, b).shape == y.shape


def test_rewire_on_moves_the_producer():
    xa = nn.Variable((2, 8))
    ya = F.relu(PF.affine(xa, 8, name='a'))
    xb = nn.Variable((2, 16))
    yb = F.relu(PF.affine(xb, 8, name='b'))
    producer = yb.parent
    xa.rewire_on(yb)
    assert xa.parent is producer and producer.outputs[0] is xa and yb.parent is None
    assert names(ya) == ['Affine', 'ReLU', 'Affine', 'ReLU']
    with pytest.raises(ValueError):
        nn.Variable((3, 3)).rewire_on(ya)


def test_recorder_classes_report_the_reference_names_and_check_shapes():
    x = nn.Variable((2, 3, 4))
    one = nn.Variable((1, 1, 1))
    for cls, two in ((qnn.MinMaxMinMaxRecorder, True), (qnn.AbsMaxRecorder, False), (qnn.MinMaxMvaRecorder, True),
                     (qnn.MaxMaxRecorder, False), (qnn.MaxMvaRecorder, False)):
        f = cls(None)
        assert f.name == cls.__name__ and f.info.type_name == cls.__name__
        y = f(x, one, one) if two else f(x, one)
        assert y.shape == x.shape and y.parent.info.type_name == cls.__name__
        with pytest.raises(ValueError):
            cls(None)(x, one) if two else cls(None)(x, one, one)
        with pytest.raises(ValueError):       # statistics must have x's rank and one element
            cls(None)(x, *([nn.Variable((1, 1))] * (2 if two else 1)))
        with pytest.raises(ValueError):
            cls(None)(x, *([nn.Variable((1, 3, 1))] * (2 if two else 1)))
    g = qnn.MinMaxMvaRecorder(None, 0.9, False)
    assert g.decay == 0.9 and g.training is False and g.clone().info == g.info
    assert qnn.MaxMvaRecorderCallback().name() == 'MaxMvaRecorder'


# ------------------------------------------------------------------------------------------------- converter driver
def test_identity_conversion_copies_the_graph_and_shares_parameters():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    y2 = GC.GraphConverter([GC.FunctionModifier()]).convert(y)
    assert y2 is not y and graph_info(y2) == graph_info(y)
    old, new = [], []
    y.visit(old.append)
    y2.visit(new.append)
    assert not set(map(id, old)) & set(map(id, new))
    for a, b in zip(old[1:], new[1:]):
        assert all(p is q for p, q in zip(a.inputs[1:], b.inputs[1:]))      # same parameter variables
    # every input of a function that starts the graph becomes an unlinked view (graph_converter.py:74-76)
    assert all(q is not p and q.parent is None and q.shape == p.shape for p, q in zip(old[0].inputs, new[0].inputs))


def test_identity_modifier_replaces_inputs():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    x2 = nn.Variable((5, 3, 8, 8))
    y2 = GC.GraphConverter([GC.IdentityModifier({x: x2})]).convert(y)
    assert names(y2) == names(y) and y2.shape == (5, 5)
    first = []
    y2.visit(first.append)
    assert first[0].inputs[0] is x2
    with pytest.raises(ValueError):
        GC.GraphConverter([GC.IdentityModifier({x: x2}, copy_value=True)]).convert(y)
    y3 = GC.GraphConverter([GC.IdentityModifier()]).convert(y)
    assert graph_info(y3) == graph_info(y)


def test_modifier_replacing_a_function_and_list_outputs():
    class ReluToPrune(GC.FunctionModifier):
        def modify(self, f, inputs):
            if f.info.type_name == 'ReLU':
                return F.prune(inputs[0], 0.5)

    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    z = F.relu(y)
    outs = GC.GraphConverter([[ReluToPrune()], GC.FunctionModifier()]).convert([y, z])
    assert isinstance(outs, list) and len(outs) == 2
    assert names(outs[1]) == [n if n != 'ReLU' else 'Prune' for n in names(z)]
    assert 'ReLU' in names(z)

    class Bad(GC.FunctionModifier):
        def modify(self, f, inputs):
            return 1

    with pytest.raises(ValueError):
        GC.GraphConverter([Bad()]).convert(y)


def test_remove_function_modifier():
    x = nn.Variable((2, 6))
    M = nn.Variable((1, 1))
    h = qnn.max_max_recorder(x, M)                      # first function of the graph
    h = PF.affine(h, 4, name='a')
    h = qnn.max_max_recorder(h, M)
    y = F.relu(h)
    bare = GC.GraphConverter([GC.RemoveFunctionModifier(rm_funcs=['MaxMaxRecorder'])]).convert(y)
    assert names(bare) == ['Affine', 'ReLU']
    assert names(y) == ['MaxMaxRecorder', 'Affine', 'MaxMaxRecorder', 'ReLU']


# ---------------------------------------------------------------------------------- float graph -> recording graph
def recording_reference(x, cfg, both=False):
    """The recording graph of small_net under the default skip lists, written out by hand."""
    act, wgt = cfg.recorder_activation, cfg.recorder_weight

    def conv_params(name):
        p = params_of(name + '/conv')
        return p['W'], p['b']

    def affine_params(name):
        p = params_of(name + '/affine')
        return p['W'], p['b']

    (w1, b1), (w2, b2) = conv_params('c1'), conv_params('c2')
    (w3, b3), (w4, b4) = affine_params('f1'), affine_params('f2')
    h = F.convolution(x, w1, b1)                        # first convolution: skipped
    with nn.parameter_scope('ref/ReLU-1'):
        h = act()(h, name='x0')
    h = F.relu(h)
    with nn.parameter_scope('ref/Convolution-2'):
        h = act()(h, name='x0')       # with BOTH: placed after the ReLU, under the same name
        w, b = wgt()(w2, name='w0'), wgt()(b2, name='w1')
    h = F.convolution(h, w, b)
    with nn.parameter_scope('ref/ReLU-3'):
        h = act()(h, name='x0')
    h = F.relu(h)
    with nn.parameter_scope('ref/Affine-4'):
        h = act()(h, name='x0')
        w, b = wgt()(w3, name='w0'), wgt()(b3, name='w1')
    h = F.affine(h, w, b)
    with nn.parameter_scope('ref/ReLU-5'):
        h = act()(h, name='x0')
    h = F.relu(h)
    if both:
        with nn.parameter_scope('ref/Affine-6'):
            h = act()(h, name='x0')
    w, b = w4, b4
    return F.affine(h, w, b)                            # last affine: skipped


def to_recording(y, cfg, training=True):
    ranks = FunctionsRankRecorder()
    y.visit(ranks)
    return GC.GraphConverter([GC.QuantizeNonQNNToRecordingModifier(ranks.functions_ranks, config=cfg,
                                                                   training=training)]).convert(y)


def test_nonqnn_to_recording_structure():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    cfg = QATConfig()
    y_rec = to_recording(y, cfg)
    assert graph_info(y_rec) == graph_info(recording_reference(x, cfg))
    # one set of statistics per recorder, under '<type>-<position>'
    keys = [k for k in nn.get_parameters(grad_only=False) if not k.startswith(('c1', 'c2', 'f1', 'f2', 'ref'))]
    assert keys == ['ReLU-1/M-x0', 'Convolution-2/M-x0', 'Convolution-2/m-w0', 'Convolution-2/M-w0',
                    'Convolution-2/m-w1', 'Convolution-2/M-w1', 'ReLU-3/M-x0', 'Affine-4/M-x0', 'Affine-4/m-w0',
                    'Affine-4/M-w0', 'Affine-4/m-w1', 'Affine-4/M-w1', 'ReLU-5/M-x0']
    assert nn.get_parameter('Affine-4/M-w0').shape == (1, 1) and nn.get_parameter('ReLU-1/M-x0').shape == (1, 1, 1, 1)
    assert names(y) == ['Convolution', 'ReLU', 'Convolution', 'ReLU', 'Affine', 'ReLU', 'Affine']   # untouched


def test_nonqnn_to_recording_positions_layers_and_flags():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    cfg = QATConfig()
    cfg.recorder_position = QATConfig.RecorderPosition.BOTH
    assert graph_info(to_recording(y, cfg)) == graph_info(recording_reference(x, cfg, both=True))
    assert 'Affine-6/M-x0' in nn.get_parameters(grad_only=False)      # the output of the last recorded function

    nn.clear_parameters()
    y = small_net(x)
    cfg = QATConfig()
    cfg.record_layers = ['Convolution', 'Affine']
    cfg.skip_inputs_layers = []
    cfg.skip_outputs_layers = []
    cfg.recorder_activation = qnn.MinMaxMvaRecorderCallback
    cfg.recorder_weight = qnn.AbsMaxRecorderCallback
    got = names(to_recording(y, cfg, training=False))
    block = ['MinMaxMvaRecorder', 'AbsMaxRecorder', 'AbsMaxRecorder']
    assert got == block + ['Convolution', 'ReLU'] + block + ['Convolution', 'ReLU'] + block + ['Affine', 'ReLU'] + \
        block + ['Affine']
    assert 'Convolution-0/m-x0' in nn.get_parameters(grad_only=False)
    rec = []
    to_recording(y, cfg, training=False).visit(rec.append)
    assert all(f.info.args['training'] is False for f in rec if f.info.type_name.endswith('Recorder'))


def test_one_recorder_for_a_variable_with_two_consumers():
    x = nn.Variable((2, 6))
    h = F.relu(PF.affine(x, 6, name='a'))
    y = F.sink(PF.affine(h, 3, name='b'), PF.affine(h, 4, name='c'), PF.affine(h, 5, name='d'))
    cfg = QATConfig()
    cfg.skip_inputs_layers, cfg.skip_outputs_layers, cfg.record_layers = [], [], ['Affine']
    got = names(to_recording(y, cfg))
    assert got.count('MaxMvaRecorder') == 2          # x and h, the latter shared by three consumers
    assert got.count('MinMaxMinMaxRecorder') == 8


def residual_net(x):
    h = F.relu(PF.convolution(x, 4, (3, 3), pad=(1, 1), name='c1'))      # Convolution-0, ReLU-1
    r = F.relu(PF.convolution(h, 4, (3, 3), pad=(1, 1), name='c2'))      # Convolution-2, ReLU-3
    return PF.affine(F.add2(h, r), 5, name='f')                          # Add2-4, Affine-5


def concat_net(x):
    a = F.relu(PF.convolution(x, 4, (3, 3), pad=(1, 1), name='c1'))      # Convolution-0, ReLU-1
    b = F.relu(PF.convolution(a, 2, (3, 3), pad=(1, 1), name='c2'))      # Convolution-2, ReLU-3
    c = F.relu(PF.convolution(b, 3, (3, 3), pad=(1, 1), name='c3'))      # Convolution-4, ReLU-5
    return PF.affine(F.concatenate(c, a, b, axis=1), 5, name='f')        # Concatenate-6, Affine-7


def find(v, type_name):
    out = []
    v.visit(lambda f: out.append(f) if f.info.type_name == type_name else None)
    return out


def test_add2_inputs_share_the_recorder_of_the_earliest_one():
    """quantize.py:110-138: h is already recorded for the second convolution ('Convolution-2/x0'); r gets a recorder
    of its own ('Add2-4/x1'), which share_recorder replaces by one on the statistics of h's."""
    x = nn.Variable((2, 3, 8, 8))
    cfg = QATConfig()
    y_rec = to_recording(residual_net(x), cfg)
    act = cfg.recorder_activation().name()
    assert names(y_rec) == ['Convolution', act, 'ReLU', act, 'MinMaxMinMaxRecorder', 'MinMaxMinMaxRecorder',
                            'Convolution', act, 'ReLU', act, 'Add2', 'Affine']
    add = find(y_rec, 'Add2')[0]
    r0, r1 = add.inputs[0].parent, add.inputs[1].parent
    assert r0.info.type_name == r1.info.type_name == act and r0 is not r1
    assert r0.inputs[1] is r1.inputs[1] is nn.get_parameter('Convolution-2/M-x0')
    conv2 = find(y_rec, 'Convolution')[1]
    assert conv2.inputs[0] is add.inputs[0]                  # one recorder on h for both of its consumers
    assert r1.inputs[0].parent.info.type_name == 'ReLU'      # r's own recorder is gone from the graph


def bias_like_residual_net(x):
    h = F.relu(PF.convolution(x, 4, (3, 3), pad=(1, 1), name='c1'))      # Convolution-0, ReLU-1
    g = F.relu(PF.convolution(x, 4, (8, 8), name='gate'))                # Convolution-2, ReLU-3: [2, 4, 1, 1]
    return PF.affine(F.add2(h, g), 5, name='f')                          # Add2-4, Affine-5


def test_add2_with_a_broadcast_operand_converts_like_any_other():
    """A residual whose second operand broadcasts over the spatial axes (a per-channel gate, [2, 4, 1, 1] onto
    [2, 4, 8, 8]): the converter does not look at shapes (quantize.py:110-138), so both inputs are recorded, the
    statistics shared are those of the input produced first, and the rewritten graph keeps the broadcast output
    shape."""
    x = nn.Variable((2, 3, 8, 8))
    cfg = QATConfig()
    y_rec = to_recording(bias_like_residual_net(x), cfg)
    act = cfg.recorder_activation().name()
    add = find(y_rec, 'Add2')[0]
    assert tuple(add.outputs[0].shape) == (2, 4, 8, 8)
    assert tuple(add.inputs[0].shape) == (2, 4, 8, 8) and tuple(add.inputs[1].shape) == (2, 4, 1, 1)
    r0, r1 = add.inputs[0].parent, add.inputs[1].parent
    assert r0.info.type_name == r1.info.type_name == act and r0 is not r1
    assert r0.inputs[1] is r1.inputs[1]                       # one set of statistics for the two operands
    set_statistics(np.random.RandomState(5))
    add_t = find(to_training(y_rec, cfg), 'Add2')[0]
    assert tuple(add_t.outputs[0].shape) == (2, 4, 8, 8)
    assert [tuple(v.shape) for v in add_t.inputs] == [(2, 4, 8, 8), (2, 4, 1, 1)]
    assert all(v.parent.info.type_name == 'DequantizeLinear' for v in add_t.inputs)


def test_share_recorder_credits_the_first_input_with_its_rank_before_the_recorder():
    """quantize.py:117-123 starts from inputs[0].rank (the first input as the float graph has it) and compares it with
    the later inputs' ranks AFTER their recorders: a later input whose recorded rank equals that figure does not
    win.  With the first input's recorded rank as the start (one higher) it would."""
    from nnabla_amd.experimental.graph_converters.quantize import _earliest

    class V(object):
        def __init__(self, rank):
            self.rank = rank
    new_inputs = [V(4), V(3)]
    assert _earliest(new_inputs, first_rank=3) == 0          # the reference's rule: 3 < 3 is false
    assert _earliest(new_inputs) == 1                        # what starting from the recorded rank would pick


def gated_net(x):
    h = F.relu(PF.convolution(x, 4, (3, 3), pad=(1, 1), name='c1'))      # Convolution-0, ReLU-1
    r = F.relu(PF.convolution(h, 4, (3, 3), pad=(1, 1), name='c2'))      # Convolution-2, ReLU-3
    return PF.affine(F.mul2(h, r), 5, name='f')                          # Mul2-4, Affine-5


def test_mul2_inputs_are_two_activations_with_recorders_of_their_own():
    """quantize.py:30-36, 148-152: both inputs of Sub2 / Mul2 / Div2 are activations and get recorders, but -- unlike
    Add2 / Concatenate (quantize.py:112-116) -- each keeps its own statistics: h the one it already has as the second
    convolution's input, r a new one named after the consumer's input ('Mul2-4/x1')."""
    x = nn.Variable((2, 3, 8, 8))
    cfg = QATConfig()
    y_rec = to_recording(gated_net(x), cfg)
    act = cfg.recorder_activation().name()
    mul = find(y_rec, 'Mul2')[0]
    r0, r1 = mul.inputs[0].parent, mul.inputs[1].parent
    assert r0.info.type_name == r1.info.type_name == act and r0 is not r1
    assert r0.inputs[1] is nn.get_parameter('Convolution-2/M-x0')
    assert r1.inputs[1] is nn.get_parameter('Mul2-4/M-x1')
    assert r1.inputs[0].parent.info.type_name == 'ReLU' and r1.inputs[0].parent.inputs[0].parent is not None


def test_concatenate_inputs_share_the_recorder_of_the_earliest_one():
    x = nn.Variable((2, 3, 8, 8))
    cfg = QATConfig()
    y_rec = to_recording(concat_net(x), cfg)
    act = cfg.recorder_activation().name()
    cat = find(y_rec, 'Concatenate')[0]
    assert tuple(cat.outputs[0].shape) == (2, 9, 8, 8)
    recs = [v.parent for v in cat.inputs]
    assert all(f.info.type_name == act for f in recs)
    # inputs (c, a, b): a is produced first and is already recorded as the input of the second convolution
    shared = nn.get_parameter('Convolution-2/M-x0')
    assert all(f.inputs[1] is shared for f in recs)
    assert recs[1] is find(y_rec, 'Convolution')[1].inputs[0].parent


def test_add2_and_concatenate_inputs_are_quantized_with_one_range():
    """quantize.py:348-373: in the training graph every input of Add2 / Concatenate goes through Q -> DQ with the
    scale and zero point of the input produced earliest."""
    for net, kind, n_in in ((residual_net, 'Add2', 2), (concat_net, 'Concatenate', 3)):
        nn.clear_parameters()
        x = nn.Variable((2, 3, 8, 8))
        cfg = QATConfig()
        y_rec = to_recording(net(x), cfg)
        set_statistics(np.random.default_rng(3))
        y_q = to_training(y_rec, cfg)
        f = find(y_q, kind)[0]
        assert len(f.inputs) == n_in
        dq = [v.parent for v in f.inputs]
        assert all(g.info.type_name == 'DequantizeLinear' for g in dq)
        assert all(g.inputs[1] is dq[0].inputs[1] and g.inputs[2] is dq[0].inputs[2] for g in dq)
        for g in dq:                       # each is the DQ of a Q with the same parameters
            q = g.inputs[0].parent
            assert q.info.type_name == 'QuantizeLinear' and q.inputs[1] is dq[0].inputs[1]
        # the output of the function is quantized for its consumer as usual
        assert f.outputs[0].function_references[0].info.type_name in ('QuantizeLinear', 'Affine')


def test_output_statistics_of_a_two_input_consumer_are_named_after_its_input_position():
    """quantize.py:233-237: the producer of Add2's second input looks its output range up as 'Add2-<rank>/x1', the
    statistics add_recorder registered for that input (quantize.py:163-164) before share_recorder rewired it."""
    x = nn.Variable((2, 3, 8, 8))
    cfg = QATConfig()
    y_rec = to_recording(residual_net(x), cfg)
    assert 'Add2-4/M-x1' in nn.get_parameters(grad_only=False)
    set_statistics(np.random.default_rng(4))
    y_q = to_training(y_rec, cfg)
    assert 'Add2-4/scale-x1' in nn.get_parameters(grad_only=False)
    assert find(y_q, 'Add2')


# ------------------------------------------------------------------------------ recording graph -> training graph
def set_statistics(rng):
    for k, v in nn.get_parameters(grad_only=False).items():
        leaf = k.split('/')[-1]
        if leaf.startswith('M-'):
            v.d = rng.uniform(0.5, 4.0)
        elif leaf.startswith('m-'):
            v.d = -rng.uniform(0.5, 4.0)


def to_training(y_rec, cfg):
    bare = GC.GraphConverter([GC.RemoveFunctionModifier(
        rm_funcs=[cfg.recorder_activation().name(), cfg.recorder_weight().name()])]).convert(y_rec)
    ranks = FunctionsRankRecorder()
    bare.visit(ranks)
    return GC.GraphConverter([GC.QuantizeRecordingToTrainingModifier(ranks.functions_ranks, config=cfg)]).convert(bare)


def training_reference(x, cfg):
    """The simulated-quantization graph of small_net, written out by hand: dequantize -> function -> quantize."""
    rm, nr, dt = cfg.round_mode, cfg.narrow_range, cfg.dtype

    def sz(scope, name):
        return nn.get_parameter('%s/scale-%s' % (scope, name)), nn.get_parameter('%s/zeropoint-%s' % (scope, name))

    def qdq(v, s, z):
        return F.dequantize_linear(F.quantize_linear(v, s, z, rm, nr, dt), s, z)

    p = params_of('c1/conv')
    h = F.convolution(x, p['W'], p['b'])
    s, z = sz('ReLU-1', 'x0')
    h = F.quantize_linear(h, s, z, rm, nr, dt)
    h = F.relu(F.dequantize_linear(h, s, z))
    s, z = sz('Convolution-2', 'x0')
    h = F.dequantize_linear(F.quantize_linear(h, s, z, rm, nr, dt), s, z)
    p = params_of('c2/conv')
    w = qdq(p['W'], *sz('Convolution-2', 'w0'))
    b = qdq(p['b'], *sz('Convolution-2', 'b'))
    h = F.convolution(h, w, b)
    s, z = sz('ReLU-3', 'x0')
    h = F.relu(F.dequantize_linear(F.quantize_linear(h, s, z, rm, nr, dt), s, z))
    s, z = sz('Affine-4', 'x0')
    h = F.dequantize_linear(F.quantize_linear(h, s, z, rm, nr, dt), s, z)
    p = params_of('f1/affine')
    w = qdq(p['W'], *sz('Affine-4', 'w0'))
    b = qdq(p['b'], *sz('Affine-4', 'b'))
    h = F.affine(h, w, b)
    s, z = sz('ReLU-5', 'x0')
    h = F.relu(F.dequantize_linear(F.quantize_linear(h, s, z, rm, nr, dt), s, z))
    p = params_of('f2/affine')
    return F.affine(h, p['W'], p['b'])


def test_recording_to_training_structure_and_scales():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    cfg = QATConfig()
    y_rec = to_recording(y, cfg)
    set_statistics(np.random.default_rng(5))
    y_q = to_training(y_rec, cfg)
    got, want = graph_info(y_q), graph_info(training_reference(x, cfg))
    assert sorted(got) == sorted(want) and len(got) == len(want)
    # forward order differs only in when parameter branches are visited; the chain of activations is the same
    main = [n for n in names(y_q)]
    assert main.count('QuantizeLinear') == 9 and main.count('DequantizeLinear') == 9
    assert main[0] == 'Convolution' and main[-1] == 'Affine'
    # every function between the skipped first and last layers reads dequantized data
    fs = []
    y_q.visit(fs.append)
    for f in fs:
        if f.info.type_name in ('ReLU', 'Convolution', 'Affine') and f is not fs[0] and f is not fs[-1]:
            assert f.inputs[0].parent.info.type_name == 'DequantizeLinear'
            assert f.inputs[0].parent.inputs[0].parent.info.type_name == 'QuantizeLinear'
    assert fs[-1].inputs[0].parent.info.type_name == 'ReLU'      # nothing was recorded for the last affine
    for f in fs:
        if f.info.type_name == 'QuantizeLinear':
            assert f.info.args == {'round_mode': 'HALF_TO_EVEN', 'narrow_range': False, 'dtype': 1}

    # scales: recorded range over 255 steps, moved to the nearest power of two; zero points are zero
    for scope, name, kind in (('ReLU-1', 'x0', 'MaxMvaRecorder'), ('Affine-4', 'w0', 'MinMaxMinMaxRecorder'),
                              ('Convolution-2', 'w1', 'MinMaxMinMaxRecorder')):
        M = nn.get_parameter('%s/M-%s' % (scope, name)).d
        m = nn.get_parameter('%s/m-%s' % (scope, name))
        want_s = oracle.recorder_scale(None if m is None else m.d, M, kind, False, 'ROUND')
        got_s = nn.get_parameter('%s/scale-%s' % (scope, name)).d
        assert got_s.shape == M.shape and np.array_equal(got_s, want_s.reshape(M.shape))
        assert np.log2(got_s.ravel()[0]) == np.round(np.log2(got_s.ravel()[0]))
        assert not nn.get_parameter('%s/zeropoint-%s' % (scope, name)).d.any()
    # the bias scale is scale(x) * scale(w), its zero point x's (quantize.py:296-327)
    sb = nn.get_parameter('Affine-4/scale-b').d
    assert sb.shape == (1,)
    assert sb[0] == nn.get_parameter('Affine-4/scale-x0').d.ravel()[0] * nn.get_parameter('Affine-4/scale-w0').d.ravel()[0]


@pytest.mark.parametrize("m, M, kind, narrow, method, want", [
    (-1.0, 1.0, 'MinMaxMinMaxRecorder', False, 'NOTROUND', 2.0 / 255),
    (-1.0, 1.0, 'MinMaxMinMaxRecorder', False, 'ROUND', 2.0 ** -7),        # log2(2/255) = -6.99
    (-1.0, 1.0, 'MinMaxMvaRecorder', False, 'CEIL', 2.0 ** -6),
    (-1.0, 1.0, 'MinMaxMvaRecorder', False, 'FLOOR', 2.0 ** -7),
    (-3.0, 3.0, 'MinMaxMinMaxRecorder', False, 'ROUND', 2.0 ** -5),        # log2(6/255) = -5.41
    (0.0, 0.0, 'MinMaxMinMaxRecorder', False, 'NOTROUND', 1e-24 / 255),   # the floor that keeps the scale positive
    (None, 63.5, 'MaxMvaRecorder', False, 'NOTROUND', 127.0 / 255),
    (None, 63.5, 'MaxMaxRecorder', False, 'ROUND', 0.5),
    (None, 127.0, 'AbsMaxRecorder', True, 'NOTROUND', 1.0),                 # narrow range: 254 steps
    (None, 127.0, 'AbsMaxRecorder', True, 'FLOOR', 1.0),
    (None, 100.0, 'AbsMaxRecorder', False, 'CEIL', 1.0),                    # 200/255 = 0.78 -> 2^0
])
def test_scale_from_statistics_known_answers(m, M, kind, narrow, method, want):
    """Closed-form cases of the scale arithmetic, for the front-end and for the oracle's restatement."""
    x = nn.Variable((2, 3))
    with nn.parameter_scope('s'):
        nn.parameter.get_parameter_or_create('M-x0', (1, 1), np.full((1, 1), M, np.float32), False)
        if m is not None:
            nn.parameter.get_parameter_or_create('m-x0', (1, 1), np.full((1, 1), m, np.float32), False)
        cb = getattr(qnn, kind + 'Callback')
        scale, zp = cb.get_scale_zeropoint(x, narrow_range=narrow, round_method=method, name='x0')
        assert cb.get_scale_zeropoint(x, name='x9') == (None, None)       # nothing recorded under that name
    assert scale.shape == (1, 1) and zp.shape == (1, 1) and zp.d[0, 0] == 0 and not scale.need_grad
    assert scale.d[0, 0] == np.float32(want) or abs(scale.d[0, 0] / np.float32(want) - 1) < 2e-7
    o = oracle.recorder_scale(m, M, kind, narrow, method)
    assert np.float32(o) == scale.d[0, 0]


# ------------------------------------------------------------------------------------------------------- scheduler
def test_scheduler_states_and_rewiring():
    x = nn.Variable((2, 3, 8, 8))
    y = small_net(x)
    tail = F.relu(y)                                    # built on y before any conversion: must follow the rewiring
    cfg = QATConfig()
    cfg.niter_to_recording, cfg.niter_to_training = 1, 3
    s = QATScheduler(cfg)
    s(y)
    s.step()
    assert s.state == QNNState.NON_QNN and len(names(tail)) == 8
    s.step()
    assert s.state == QNNState.RECORDING
    assert names(tail) == names(recording_reference(x, cfg)) + ['ReLU']
    set_statistics(np.random.default_rng(1))
    s.step()
    assert s.state == QNNState.RECORDING
    s.step()
    assert s.state == QNNState.TRAINING
    got = names(tail)
    assert got[-1] == 'ReLU' and got.count('QuantizeLinear') == 9 and not any(n.endswith('Recorder') for n in got)
    assert y.shape == (2, 5)
    for _ in range(3):
        s.step()
    assert s.state == QNNState.TRAINING and names(tail) == got


def test_scheduler_refuses_batch_normalization_folding():
    """bn_folding / bn_self_folding (qnn.py:842-856) with a BatchNormalization in the graph: refused, not ignored."""
    import types

    class Graph(object):
        def visit(self, fn):
            fn(types.SimpleNamespace(info=types.SimpleNamespace(type_name='BatchNormalization')))

    cfg = qnn.QATTensorRTConfig()
    cfg.niter_to_recording, cfg.niter_to_training = 0, 5
    sched = QATScheduler(cfg)
    sched(Graph())
    with pytest.raises(NotImplementedError):
        sched.step()
    cfg.bn_folding = cfg.bn_self_folding = False
    sched = QATScheduler(cfg)
    sched._refuse_bn_folding(Graph())        # nothing to fold: no complaint


def test_scheduler_argument_checks():
    cfg = QATConfig()
    with pytest.raises(ValueError):
        QATScheduler(cfg)                               # niter_to_training defaults to -1
    cfg.niter_to_recording, cfg.niter_to_training = 5, 5
    with pytest.raises(ValueError):
        QATScheduler(cfg)
    cfg.niter_to_recording = -1
    with pytest.raises(ValueError):
        QATScheduler(cfg)
    cfg.niter_to_recording, cfg.niter_to_training = 0, 2
    cfg.precision_mode = qnn.PrecisionMode.QNN
    with pytest.raises(NotImplementedError):
        GC.QuantizeRecordingToTrainingModifier({}, config=cfg)


# ------------------------------------------------------------------------------------------- pins of the oracle
def test_oracle_recorder_pins():
    """What fixes ``oracle.range_recorder`` independently of its own text: running extrema are the extrema of
    everything seen (and of the starting value), a moving average fed a constant follows c (1 - decay^n) -- swapped
    weights or a dropped term fail it at n = 1 -- and one step from zero gives the fp32 nearest to the double
    1 - decay (MulScalar casts its Python float once, mul_scalar.hpp), not 1 minus the fp32 decay."""
    rng = np.random.default_rng(9)
    batches = [rng.standard_normal((5, 7, 3)).astype(np.float32) * (k + 1) for k in range(4)]
    m = M = A = X = np.float32(0)
    for k, x in enumerate(batches):
        m, M = oracle.range_recorder(x, m, M, 'MinMaxMinMaxRecorder')
        _, A = oracle.range_recorder(x, None, A, 'AbsMaxRecorder')
        _, X = oracle.range_recorder(x, None, X, 'MaxMaxRecorder')
        seen = np.concatenate([b.ravel() for b in batches[:k + 1]] + [np.zeros(1, np.float32)])
        assert (m, M, A, X) == (seen.min(), seen.max(), np.abs(seen).max(), seen.max())
    neg = -np.abs(batches[0]) - 1
    assert oracle.range_recorder(neg, None, np.float32(0), 'MaxMaxRecorder')[1] == 0       # the start value wins
    assert oracle.range_recorder(neg, None, np.float32(-9), 'MaxMaxRecorder')[1] == neg.max()
    assert oracle.range_recorder(neg, None, np.float32(0), 'AbsMaxRecorder')[1] == -neg.min()

    x = np.full((3, 4), 0.25, np.float32)
    x[1, 2], x[2, 0] = 5.0, -2.0
    for decay in (0.9, 0.75, 0.99):
        lo = hi = one = np.float32(0)
        for n in range(1, 30):
            lo, hi = oracle.range_recorder(x, lo, hi, 'MinMaxMvaRecorder', decay)
            _, one = oracle.range_recorder(x, None, one, 'MaxMvaRecorder', decay)
            assert abs(hi - 5.0 * (1 - decay ** n)) < 2e-6 * n and abs(lo + 2.0 * (1 - decay ** n)) < 2e-6 * n
            assert one == hi
    unit = np.ones((2, 2), np.float32)
    got = oracle.range_recorder(unit, None, np.float32(0), 'MaxMvaRecorder', 0.99)[1]
    assert np.float32(got).view(np.uint32) == 0x3c23d70a                 # fp32(0.01); 1 - fp32(0.99) is 0x3c23d700
    assert np.float32(1) - np.float32(0.99) != got
    # from a non-zero start: two products rounded to fp32, then their sum
    got = oracle.range_recorder(3 * unit, None, np.float32(7), 'MaxMvaRecorder', 0.9)[1]
    assert got == np.float32(np.float32(np.float32(0.9) * np.float32(7)) + np.float32(np.float32(1.0 - 0.9) * np.float32(3)))
    assert abs(got - 6.6) < 1e-6
