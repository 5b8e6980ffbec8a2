"""Rebuilding a graph function by function (mirrors experimental/graph_converters/graph_converter.py:21-229).

``GraphConverter(modifiers).convert(y)`` walks the graph that produces ``y`` in forward order, once per modifier.
For every function the modifier is handed the function and the *new* variables that stand for its inputs, and
returns the new variable that stands for its output (or None: the function is re-created unchanged on the new
inputs).  The original graph is left intact; parameters are shared between both.
"""
from collections import defaultdict

from ... import functions as F
from ...variable import Variable


class FunctionModifier(object):
    """Base class: override ``modify(f, inputs)``."""

    def __init__(self):
        self._map_func_inputs = defaultdict(list)   # function of the old graph -> its inputs in the new graph
        self.outputs = None

    def init_map_func_inputs(self, f, inputs):
        self._map_func_inputs[f] = inputs

    def get_parameter_scope(self, v):
        """Scope path under which variable ``v`` is registered as a parameter ('' if it is not)."""
        from ... import parameter
        for key, p in parameter.get_parameters().items():
            if p is v:
                return '/'.join(key.split('/')[:-1])
        return ''

    def _force_list(self, o):
        if isinstance(o, tuple):
            return list(o)
        return o if isinstance(o, list) else [o]

    def _copy_inputs(self, inputs):
        """Unlinked views of graph inputs: same arrays, no producing function."""
        return [i.get_unlinked_variable(need_grad=i.need_grad) for i in inputs]

    def __call__(self, f):
        known = f in self._map_func_inputs
        if f.inputs[0].parent is None and not known:
            self._map_func_inputs[f] = self._copy_inputs(f.inputs)
        inputs = self._map_func_inputs[f]
        # inputs nothing upstream has replaced (parameters, other leaves) are used as they are
        if len(f.inputs) > 1:
            for i, orig in enumerate(f.inputs):
                if i >= len(inputs):
                    inputs.append(orig)
                elif inputs[i] is None:
                    inputs[i] = orig

        o = self.modify(f, inputs)
        if not isinstance(o, (type(None), Variable)):
            raise ValueError('Return None or nn.Variable')
        if o is None:
            o = self._modify_as_same(f, inputs)
        outputs = self._force_list(o)
        self.outputs = outputs

        # hand the new outputs to the functions that consume the old ones
        for old, new in zip(f.outputs, outputs):
            consumers = old.function_references
            if not consumers:
                return
            for g in consumers:
                slots = self._map_func_inputs[g]
                if not slots:
                    slots.extend([None] * len(g.inputs))
                for i, inp in enumerate(g.inputs):
                    if inp is old:
                        slots[i] = new

    def modify(self, f, inputs):
        """Returns the variable replacing ``f``'s output, built on ``inputs``, or None to keep ``f`` as it is."""
        return None

    def _modify_as_same(self, f, inputs):
        return f.function.clone()(*inputs)

    def _call_function(self, type_name, inputs, args):
        """A function named as in ``F`` applied to ``inputs`` with keyword arguments ``args``."""
        import re
        snake = re.sub(r'(?<=[a-z0-9])([A-Z])', r'_\1', type_name).lower()
        table = {'inqaffine': 'inq_affine', 'inqconvolution': 'inq_convolution', 're_lu': 'relu'}
        fn = getattr(F, table.get(snake, snake))
        return fn(*inputs, **args)

    def __finish__(self):
        """Called once after a whole graph has been converted."""

    def finish_up(self):
        self._map_func_inputs = defaultdict(list)
        self.__finish__()


class GraphConverter(object):
    """Applies modifiers (a list, possibly nested) one after the other, each to the result of the previous one."""

    def __init__(self, modifiers=[]):
        self._modifiers = self._flatten(modifiers)

    def _flatten(self, modifiers):
        flat = []
        for m in modifiers:
            flat += self._flatten(m) if isinstance(m, list) else [m]
        return flat

    def convert(self, o):
        """``o``: an output variable or a list of them; returns the converted counterpart(s)."""
        as_list = isinstance(o, list)
        outputs = list(o) if isinstance(o, (list, tuple)) else [o]
        for modifier in self._modifiers:
            end = F.sink(*outputs)          # one terminal node, so that a single traversal reaches every output
            end.visit(modifier)
            outputs = list(modifier.outputs[0].parent.inputs)
            modifier.finish_up()
        return outputs if as_list else outputs[0]
