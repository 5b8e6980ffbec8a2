"""Quantization-aware training on the hip context: range recorders, the QAT configuration and the scheduler that
moves a network NON_QNN -> RECORDING -> TRAINING (mirrors python/src/nnabla/utils/qnn.py).

The recorders are identity functions that track the range of what flows through them.  The reference writes them
as PythonFunctions over Min / Max / Abs / Maximum2 helper functions (qnn.py:42-560); here each one is the registry
function ``RangeRecorder`` of the hip extension (one scan kernel), reporting the reference class's name so that
the graph converters recognise it by ``info.type_name``.

Not carried over: batch-normalisation folding (``bn_folding`` / ``bn_self_folding`` are accepted and have nothing to
act on, since no BatchNormalization function exists on this path) and re-registering parameters with a solver.
"""
from collections import OrderedDict
from enum import Enum

import numpy as np

from .. import parameter as _parameter
from ..function import Function
from ..initializer import ConstantInitializer

_MODES = {"MinMaxMinMaxRecorder": 0, "AbsMaxRecorder": 1, "MinMaxMvaRecorder": 2, "MaxMaxRecorder": 3,
          "MaxMvaRecorder": 4}

__round_methods__ = {'CEIL': np.ceil, 'ROUND': np.round, 'FLOOR': np.floor, 'NOTROUND': None}


class _Recorder(Function):
    """Base of the five recorder function classes: ``cls(ctx, [decay,] training)`` then ``f(x, [m,] M)``."""
    _moving_average = False

    def __init__(self, ctx=None, *args, **kw):
        names = (("decay", 0.99), ("training", True)) if self._moving_average else (("training", True),)
        vals = dict(names)
        for (k, _), v in zip(names, args):
            vals[k] = v
        vals.update(kw)
        self.training = bool(vals["training"])
        self.decay = float(vals.get("decay", 0.99))
        args_ = dict(training=self.training)
        if self._moving_average:
            args_["decay"] = self.decay
        Function.__init__(self, "RangeRecorder", ctx, [_MODES[type(self).__name__], int(self.training)],
                          [self.decay], args=args_)

    def clone(self, ctx=None):
        return type(self)(ctx, **self.info.args)


class MinMaxMinMaxRecorder(_Recorder):
    """m = min(m, min x), M = max(M, max x) over the training iterations (qnn.py:42-97)."""


class AbsMaxRecorder(_Recorder):
    """M = max(M, max |x|) (qnn.py:148-201)."""


class MinMaxMvaRecorder(_Recorder):
    """Moving averages of the batch minimum and maximum: m = decay m + (1 - decay) min x (qnn.py:255-313)."""
    _moving_average = True


class MaxMaxRecorder(_Recorder):
    """M = max(M, max x) (qnn.py:381-433)."""


class MaxMvaRecorder(_Recorder):
    """Moving average of the batch maximum: M = decay M + (1 - decay) max x (qnn.py:478-531)."""
    _moving_average = True


def minmax_minmax_recorder(x, m, M, training=True):
    return MinMaxMinMaxRecorder(None, training)(x, m, M)


def abs_max_recorder(x, M, training=True):
    return AbsMaxRecorder(None, training)(x, M)


def minmax_mva_recorder(x, m, M, decay=0.99, training=True):
    return MinMaxMvaRecorder(None, decay, training)(x, m, M)


def max_max_recorder(x, M, training=True):
    return MaxMaxRecorder(None, training)(x, M)


def max_mva_recorder(x, M, decay=0.99, training=True):
    return MaxMvaRecorder(None, decay, training)(x, M)


def _int8_levels(narrow_range):
    """Number of steps of the int8 grid: 255, or 254 when -128 is left out."""
    return 254 if narrow_range else 255


def _pow2_scale(scale, round_method):
    """The scale moved to a power of two, the exponent rounded as ``round_method`` says (qnn.py:136-139)."""
    rnd = __round_methods__[round_method]
    if rnd is None:
        return scale
    return 2 ** rnd(np.log(scale) / np.log(2))


def _register_scale(scale, like, name):
    """Registers 'scale-<name>' and an all-zero 'zeropoint-<name>' in the current scope (qnn.py:141-147)."""
    zp = np.round((np.zeros_like(like) / scale).astype(np.int8))
    zp = _parameter.get_parameter_or_create('zeropoint-{}'.format(name), zp.shape, zp, False)
    scale = np.asarray(scale)
    scale = _parameter.get_parameter_or_create('scale-{}'.format(name), scale.shape, scale, False)
    return scale, zp


class _Callback(object):
    """What ``QATConfig.recorder_activation`` / ``recorder_weight`` hold: calling an instance puts a recorder on
    ``x`` with its statistics registered as parameters of the current scope; ``get_scale_zeropoint`` (called on the
    class) turns the recorded statistics into QuantizeLinear parameters."""
    _two_sided = False
    _function = None

    def name(self):
        n = type(self).__name__
        return n[:n.rfind('Callback')]

    def __call__(self, x, axes=[1], training=True, name=''):
        shape = [1] * x.ndim
        stats = []
        if self._two_sided:
            stats.append(_parameter.get_parameter_or_create('m-{}'.format(name), shape, ConstantInitializer()))
        stats.append(_parameter.get_parameter_or_create('M-{}'.format(name), shape, ConstantInitializer()))
        return type(self)._function(x, *stats, training=training)

    @classmethod
    def get_scale_zeropoint(cls, x, axes=[1], narrow_range=False, round_method='NOTROUND', name=''):
        """(scale, zero point) parameters for ``x`` from the statistics recorded under ``name`` in the current scope,
        or (None, None) where no recorder was placed."""
        M = _parameter.get_parameter('M-{}'.format(name))
        m = _parameter.get_parameter('m-{}'.format(name)) if cls._two_sided else None
        if cls._two_sided:
            if M is None and m is None:
                return None, None
            shape = [1] * x.ndim
            m = _parameter.get_parameter_or_create('m-{}'.format(name), shape)
            M = _parameter.get_parameter_or_create('M-{}'.format(name), shape)
            # the recorded width spread over the grid; 1e-24 keeps the scale off zero (qnn.py:131-134, :360-363)
            scale = np.maximum(M.d - m.d, 1e-24) / _int8_levels(narrow_range)
        else:
            if M is None:
                return None, None
            scale = (2 * M.d) / _int8_levels(narrow_range)   # symmetric range [-M, M] (qnn.py:236, :465, :548)
        scale = _pow2_scale(scale, round_method)
        return _register_scale(scale, M.d, name)


class MinMaxMinMaxRecorderCallback(_Callback):
    _two_sided = True
    _function = staticmethod(minmax_minmax_recorder)


class AbsMaxRecorderCallback(_Callback):
    _function = staticmethod(abs_max_recorder)


class MinMaxMvaRecorderCallback(_Callback):
    _two_sided = True
    _function = staticmethod(minmax_mva_recorder)


class MaxMaxRecorderCallback(_Callback):
    _function = staticmethod(max_max_recorder)


class MaxMvaRecorderCallback(_Callback):
    _function = staticmethod(max_mva_recorder)


class PrecisionMode(Enum):
    QNN = 0
    SIM_QNN = 1
    MIXED_QNN = 2


class QNNState(Enum):
    NON_QNN = 0
    RECORDING = 1
    TRAINING = 2
    DEPLOYMENT = 3


class QATConfig(object):
    """Settings of quantization-aware training (qnn.py:627-740); the defaults are the reference's except
    ``ext_name``."""

    class RoundingMethod(Enum):
        CEIL = 'CEIL'
        ROUND = 'ROUND'
        FLOOR = 'FLOOR'
        NOTROUND = 'NOTROUND'

    class RecorderPosition(Enum):
        BEFORE = 0
        BOTH = 1

    ext_name = "hip"
    zero_point = False
    dtype = np.int8
    precision_mode = PrecisionMode.SIM_QNN
    channel_last = False
    channel_wise = False
    niter_to_recording = 0
    niter_to_training = -1
    pow2 = RoundingMethod.ROUND
    narrow_range = False
    round_mode = 'HALF_TO_EVEN'
    bn_folding = False
    bn_self_folding = False
    recorder_weight = MinMaxMinMaxRecorderCallback
    recorder_activation = MaxMvaRecorderCallback
    record_layers = []
    recorder_position = RecorderPosition.BEFORE
    skip_inputs_layers = ['Convolution', 'Deconvolution']
    skip_outputs_layers = ['Affine']
    learning_rate_scale = 0.1
    skip_bias = False


class QATTensorRTConfig(QATConfig):
    pow2 = QATConfig.RoundingMethod.ROUND
    bn_folding = True
    bn_self_folding = True
    record_layers = ["Convolution", "Deconvolution", "Affine", "BatchMatmul", "ReLU"]
    record_position = QATConfig.RecorderPosition.BEFORE


qat_default_config = QATTensorRTConfig()


class FunctionsRankRecorder(object):
    """``pred.visit(recorder)`` numbers the functions of a graph in forward order; the numbers name the parameter
    scopes of the recorders ('Affine-3/...') and so tie the recording graph to the training graph
    (qnn.py:753-763)."""

    def __init__(self, functions_only_for_training=['ImageAugmentation', 'Dropout']):
        self.functions_only_for_training = functions_only_for_training
        self.rank = 0
        self.functions_ranks = {}

    def __call__(self, f):
        if f.info.type_name in self.functions_only_for_training:
            return
        self.functions_ranks[f] = self.rank
        self.rank += 1


class QATScheduler(object):
    """Registers network outputs and rewires them as training proceeds: at step ``niter_to_recording`` recorders are
    inserted, at step ``niter_to_training`` they are replaced by QuantizeLinear / DequantizeLinear pairs with the
    recorded scales (qnn.py:766-925)."""

    def __init__(self, config=qat_default_config, solver=None):
        if config.niter_to_training <= 0 or config.niter_to_recording < 0:
            raise ValueError('niter_to_recording must be at least 0 and niter_to_training greater than 0.')
        if config.niter_to_training - config.niter_to_recording <= 0:
            raise ValueError('niter_to_training must come after niter_to_recording.')
        self.config = config
        self.solver = solver
        self.counter = 0
        self.state = QNNState.NON_QNN
        self.registry = []

    def __call__(self, pred, training=True):
        self.registry.append((pred, training))

    def _refuse_bn_folding(self, pred):
        """BatchNormalization folding (qnn.py:842-856) is not part of this build: a graph that would need it is refused
        rather than converted with unfolded statistics."""
        if not (self.config.bn_folding or self.config.bn_self_folding):
            return
        found = []
        pred.visit(lambda f: found.append(f) if f.info.type_name == 'BatchNormalization' else None)
        if found:
            raise NotImplementedError("QATScheduler: bn_folding / bn_self_folding is set and the network holds a "
                                      "BatchNormalization; BatchNormalization folding is not available.")

    def _schedule_to_recording(self):
        from ..experimental import graph_converters as GC
        for i, (pred, training) in enumerate(self.registry):
            self._refuse_bn_folding(pred)
            ranks = FunctionsRankRecorder()
            pred.visit(ranks)
            converted = GC.GraphConverter([GC.QuantizeNonQNNToRecordingModifier(
                ranks.functions_ranks, config=self.config, training=training)]).convert(pred)
            pred.rewire_on(converted)
            pred.need_grad = False
            self.registry[i] = (pred, training)
        self.state = QNNState.RECORDING

    def _schedule_to_training(self):
        from ..experimental import graph_converters as GC
        cfg = self.config
        for i, (pred, training) in enumerate(self.registry):
            bare = GC.GraphConverter([GC.RemoveFunctionModifier(
                rm_funcs=[cfg.recorder_activation().name(), cfg.recorder_weight().name()])]).convert(pred)
            pred.rewire_on(bare)
            ranks = FunctionsRankRecorder()
            pred.visit(ranks)
            converted = GC.GraphConverter([GC.QuantizeRecordingToTrainingModifier(
                ranks.functions_ranks, config=cfg)]).convert(pred)
            pred.rewire_on(converted)
            self.registry[i] = (pred, training)
        if self.solver is not None:
            self.solver.set_learning_rate(self.solver.learning_rate() * cfg.learning_rate_scale)
        self.state = QNNState.TRAINING

    def step(self):
        """One training iteration has passed; converts the registered graphs when a boundary is reached."""
        if self.counter == self.config.niter_to_recording:
            self._schedule_to_recording()
        elif self.counter == self.config.niter_to_training:
            self._schedule_to_training()
        self.counter += 1

    def save(self, fname, inputs, batch_size=1, net_name='net', deploy=False):
        """Writes the registered evaluation network(s) (those registered with ``training=False``) as an NNP file with
        inputs 'x0', 'x1', ... and outputs 'y0', 'y1', ... (qnn.py:927-1000).  ``deploy=True`` is not available (it
        is not in the reference either)."""
        if deploy:
            raise NotImplementedError("QATScheduler.save: deployment conversion is not supported.")
        from .save import save
        inputs = list(inputs) if isinstance(inputs, (list, tuple)) else [inputs]
        for pred, training in self.registry:
            if training:
                continue
            outputs = list(pred) if isinstance(pred, (list, tuple)) else [pred]
            names = OrderedDict(('x{}'.format(i), v) for i, v in enumerate(inputs))
            outs = OrderedDict(('y{}'.format(i), v) for i, v in enumerate(outputs))
            save(fname, {'networks': [{'name': net_name, 'batch_size': batch_size, 'outputs': outs, 'names': names}],
                         'executors': [{'name': 'runtime', 'network': net_name, 'data': list(names),
                                        'output': list(outs)}]})
