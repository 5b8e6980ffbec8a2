"""The two graph rewrites of quantization-aware training (mirrors experimental/graph_converters/quantize.py).

``QuantizeNonQNNToRecordingModifier`` puts range recorders in front of the functions of a float network;
``QuantizeRecordingToTrainingModifier`` (on the graph with the recorders taken out again) wraps every function in
QuantizeLinear -> DequantizeLinear pairs whose scales come from the recorded ranges.  Both find their parameters
under the scope '<function type>-<position of the function in the graph>'.

The inputs of Add2 and Concatenate share one recorder and one quantization range (that of the input produced
earliest in the graph), as in the reference; both inputs of Add2, Sub2, Mul2, Div2 and Pow2 are activations
(quantize.py:30-36), and all five exist on the hip context, broadcasting included.  The QNN / MIXED_QNN precision
modes are None in the reference too (quantize.py:409-413).
"""
from collections import defaultdict

import numpy as np

from ... import functions as F
from ... import parameter
from .graph_converter import FunctionModifier

_WITH_BIAS = ('Affine', 'Convolution', 'Deconvolution', 'DepthwiseConvolution', 'DepthwiseDeconvolution')


def _scope_of(f, ranks):
    return '{}-{}'.format(f.info.type_name, ranks.get(f, -1))


# the functions whose two inputs are both activations (quantize.py:30-36)
_TWO_ACTIVATIONS = ('Add2', 'Sub2', 'Mul2', 'Div2', 'Pow2')
# the functions whose inputs have to share one quantization range (quantize.py:112-116, 351-353)
_SHARED_RANGE = ('Add2', 'Concatenate')


def _count_activations(f, inputs):
    """How many leading inputs of ``f`` are activations; the rest are parameters (quantize.py:148-152)."""
    fn = f.info.type_name
    if fn in ('Concatenate', 'Stack'):
        return len(inputs)
    return 2 if fn in _TWO_ACTIVATIONS else 1


def _earliest(variables, eligible=lambda v: True, first_rank=None):
    """Index of the variable of lowest rank (first of equals) among the eligible ones after the first, which is the
    candidate to beat (quantize.py:117-123, 354-360).  ``first_rank``: the rank that candidate is credited with when
    it is not its own (the recording pass compares the later inputs' recorded ranks with the rank of the first
    input BEFORE its recorder, quantize.py:120)."""
    idx, low = 0, (variables[0].rank if first_rank is None else first_rank)
    for i, v in enumerate(variables[1:]):
        if eligible(v) and v.rank < low:
            idx, low = i + 1, v.rank
    return idx


def _axes(cfg):
    return [3] if cfg.channel_last else [1]


class QuantizeNonQNNToRecordingModifier(FunctionModifier):
    """Float graph -> recording graph (quantize.py:26-229)."""

    def __init__(self, functions_ranks, config=None, training=True):
        super(QuantizeNonQNNToRecordingModifier, self).__init__()
        self._config = config
        self._training = training
        self.functions_ranks = functions_ranks

    def get_function_rank(self, f):
        return self.functions_ranks.get(f, -1)

    # -- which functions get recorders (quantize.py:45-108)
    @staticmethod
    def _types_upstream(f):
        seen, todo, names = set(), [f], set()
        while todo:
            g = todo.pop()
            for v in g.inputs:
                p = v.parent
                if p is not None and id(p) not in seen:
                    seen.add(id(p))
                    names.add(p.info.type_name)
                    todo.append(p)
        return names

    @staticmethod
    def _types_downstream(f):
        seen, todo, names = set(), [f], set()
        while todo:
            g = todo.pop()
            for c in g.outputs[0].function_references:
                if id(c) not in seen:
                    seen.add(id(c))
                    names.add(c.info.type_name)
                    todo.append(c)
        return names

    def _is_skipped(self, f):
        """The first layers of the types in ``skip_inputs_layers`` (nothing of such a type upstream) and the last
        layers of the types in ``skip_outputs_layers`` (nothing of such a type downstream) stay in float."""
        cfg, fn = self._config, f.info.type_name
        if cfg.skip_inputs_layers and fn in cfg.skip_inputs_layers:
            if not (self._types_upstream(f) & set(cfg.skip_inputs_layers)):
                return True
        if cfg.skip_outputs_layers and fn in cfg.skip_outputs_layers:
            if not (self._types_downstream(f) & set(cfg.skip_outputs_layers)):
                return True
        return False

    def check(self, f):
        fn, cfg = f.info.type_name, self._config
        if fn in ('Sink', 'BatchNormalization'):
            return False
        if cfg.record_layers and fn not in cfg.record_layers:
            return False
        return not self._is_skipped(f)

    # -- quantize.py:140-181
    def add_recorder(self, f, inputs, cfg):
        scope = _scope_of(f, self.functions_ranks)
        act, wgt = cfg.recorder_activation, cfg.recorder_weight
        n_act = _count_activations(f, inputs)
        out = []
        for i, v in enumerate(inputs[:n_act]):
            taken = v.function_references
            if taken and taken[0].info.type_name == act().name():
                v = taken[0].outputs[0]          # another consumer already records this variable
            elif not (v.parent is not None and v.parent.info.type_name == act().name()):
                with parameter.parameter_scope(scope):
                    v = act()(v, axes=_axes(cfg), training=self._training, name='x{}'.format(i))
            out.append(v)
        for i, p in enumerate(inputs[n_act:]):
            with parameter.parameter_scope(scope):
                out.append(wgt()(p, axes=_axes(cfg), training=self._training, name='w{}'.format(i)))
        return out

    # -- quantize.py:110-138
    def share_recorder(self, f, inputs, new_inputs, cfg):
        """Add2 / Concatenate: every input is recorded by the recorder (the statistics) of the input that is produced
        earliest; the other inputs' own recorders are taken out again."""
        if f.info.type_name not in _SHARED_RANGE:
            return new_inputs
        idx = _earliest(new_inputs, first_rank=inputs[0].rank)
        scope = self.get_parameter_scope(new_inputs[idx].parent.inputs[1])
        for i, v in enumerate(new_inputs):
            if i == idx:
                continue
            v = v.parent.inputs[0]
            with parameter.parameter_scope(scope):
                v = cfg.recorder_activation()(v, axes=_axes(cfg), training=self._training, name='x0')
            new_inputs[i] = v
        return new_inputs

    def modify(self, f, inputs):
        if not self.check(f):
            return None
        cfg = self._config
        new_inputs = self.share_recorder(f, inputs, self.add_recorder(f, inputs, cfg), cfg)
        h = self._modify_as_same(f, new_inputs)
        if cfg.recorder_position == cfg.RecorderPosition.BOTH:
            # also record the output, under the scope of the (first) function that consumes it
            nxt = f.outputs[0].function_references[0]
            with parameter.parameter_scope(_scope_of(nxt, self.functions_ranks)):
                h = cfg.recorder_activation()(h, axes=_axes(cfg), training=self._training, name='x0')
        return h


class QuantizeRecordingToTrainingModifier(FunctionModifier):
    """Recorder-free graph + recorded ranges -> simulated-quantization graph (quantize.py:232-430)."""

    class SimulatedQNN(object):
        """inputs -> Q -> DQ -> function -> Q; the DQ of an output is added by whoever consumes it."""

        def __init__(self, functions_ranks, modifier=None, config=None):
            self._config = config
            self._modifier = modifier
            self._map_input_scale_zeropoint = defaultdict(list)
            self.functions_ranks = functions_ranks

        def get_function_rank(self, f):
            return self.functions_ranks.get(f, -1)

        def try_to_quantize(self, x, scale, zero_point, round_mode, narrow_range, dtype):
            if scale is None:
                return x
            return F.quantize_linear(x, scale, zero_point, round_mode, narrow_range, dtype)

        def try_to_dequantize(self, x, scale, zero_point):
            return x if scale is None else F.dequantize_linear(x, scale, zero_point)

        def get_quantization_params(self, variable):
            p = variable.parent
            if p is not None and p.info.type_name == 'QuantizeLinear':
                return p.inputs[1].d, p.inputs[2].d
            return None, None

        def _q(self, v, scale, zp):
            cfg = self._config
            return self.try_to_quantize(v, scale, zp, cfg.round_mode, cfg.narrow_range, cfg.dtype)

        # quantize.py:296-327: the bias is quantized with scale(x) * scale(w) and x's zero point
        def requantize_bias(self, f, inputs, scope, skip_bias=False):
            if f.info.type_name not in _WITH_BIAS or len(inputs) != 3:
                return inputs
            x, w, b = inputs
            sx, zpx = self.get_quantization_params(x)
            sw, _ = self.get_quantization_params(w)
            if sx is None or sw is None:
                return inputs
            sbd = np.reshape(sx.copy(), (1,)) * np.reshape(sw.copy(), (1,))
            with parameter.parameter_scope(scope):
                sb = parameter.get_parameter_or_create('scale-b', (1,), sbd, False)
                zpb = parameter.get_parameter_or_create('zeropoint-b', (1,), np.reshape(zpx.copy(), (1,)), False)
            if b.parent is not None and b.parent.info.type_name == 'QuantizeLinear':
                b = b.parent.inputs[0]
                if not skip_bias:
                    b = self._q(b, sb, zpb)
                inputs[2] = b
            return inputs

        # quantize.py:329-358
        def quantize_inputs(self, f, inputs, scope):
            cfg = self._config
            nr, pow2 = cfg.narrow_range, cfg.pow2.value
            n_act = _count_activations(f, inputs)
            out = []
            for i, v in enumerate(inputs[:n_act]):
                if v.rank == 0:      # a graph input; everything else was quantized where it was produced
                    with parameter.parameter_scope(scope):
                        s, zp = cfg.recorder_activation.get_scale_zeropoint(
                            v, axes=_axes(cfg), narrow_range=nr, round_method=pow2, name='x{}'.format(i))
                    v = self._q(v, s, zp)
                    self._map_input_scale_zeropoint[v] = (s, zp)
                out.append(v)
            for i, p in enumerate(inputs[n_act:]):
                with parameter.parameter_scope(scope):
                    s, zp = cfg.recorder_weight.get_scale_zeropoint(
                        p, axes=_axes(cfg), narrow_range=nr, round_method=pow2, name='w{}'.format(i))
                out.append(self._q(p, s, zp))
            return self.requantize_bias(f, out, scope, cfg.skip_bias)

        # quantize.py:360-373
        def dequantize_inputs(self, inps):
            for i, v in enumerate(inps):
                for c in v.function_references:
                    if c.info.type_name == 'DequantizeLinear':
                        v = c.outputs[0]       # already dequantized for another consumer
                        break
                if v.parent is not None and v.parent.info.type_name == 'QuantizeLinear':
                    v = self.try_to_dequantize(v, v.parent.inputs[1], v.parent.inputs[2])
                inps[i] = v
            return inps

        # quantize.py:348-373
        def shared_quantization(self, f, inps):
            """Add2 / Concatenate: every input is quantized with the scale and zero point of the (dequantized) input
            that is produced earliest."""
            if f.info.type_name not in _SHARED_RANGE:
                return inps

            def dequantized(v):
                return v.parent is not None and v.parent.info.type_name == 'DequantizeLinear'

            idx = _earliest(inps, dequantized)
            s = zp = None
            if dequantized(inps[idx]):
                s, zp = inps[idx].parent.inputs[1:3]
            for i in range(len(inps)):
                if i == idx:
                    continue
                v = inps[i]
                if dequantized(v):
                    v = v.parent.inputs[0].parent.inputs[0]      # back to the value before its own Q -> DQ
                inps[i] = self.try_to_dequantize(self._q(v, s, zp), s, zp)
            return inps

        # quantize.py:240-271
        def _quantize_outputs(self, f, h):
            cfg = self._config
            s = zp = None
            for nxt in f.outputs[0].function_references:
                if nxt.info.type_name == 'Sink':
                    return h
                name = 'x0'
                if nxt.info.type_name in _TWO_ACTIVATIONS:      # recorded as the consumer's i-th input
                    for i, v in enumerate(nxt.inputs):
                        if v is f.outputs[0]:
                            name = 'x{}'.format(i)
                with parameter.parameter_scope(_scope_of(nxt, self.functions_ranks)):
                    s, zp = cfg.recorder_activation.get_scale_zeropoint(
                        h, axes=_axes(cfg), narrow_range=cfg.narrow_range, round_method=cfg.pow2.value, name=name)
                if s is not None:
                    break
            h = self._q(h, s, zp)
            self._map_input_scale_zeropoint[h] = (s, zp)
            return h

        def modify(self, f, inputs):
            scope = _scope_of(f, self.functions_ranks)
            inps = self.dequantize_inputs(self.quantize_inputs(f, inputs, scope))
            inps = self.shared_quantization(f, inps)
            h = self._modifier._modify_as_same(f, inps)
            if f.info.type_name == 'Sink':
                return h
            return self._quantize_outputs(f, h)

        def __finish__(self):
            self._map_input_scale_zeropoint = defaultdict(list)

    def __init__(self, functions_ranks, config=None):
        super(QuantizeRecordingToTrainingModifier, self).__init__()
        from ...utils.qnn import PrecisionMode
        if config.precision_mode != PrecisionMode.SIM_QNN:
            raise NotImplementedError("only PrecisionMode.SIM_QNN is available (as in the reference).")
        self._mode = self.SimulatedQNN(functions_ranks, self, config)

    def modify(self, f, inputs):
        return self._mode.modify(f, inputs)

    def __finish__(self):
        self._mode.__finish__()
