"""Removing functions from a graph (mirrors experimental/graph_converters/remove_function.py:18-63)."""
from .graph_converter import FunctionModifier


class RemoveFunctionModifier(FunctionModifier):
    """Drops every function whose type name is in ``rm_funcs``: its consumers read its first input instead."""

    def __init__(self, rm_funcs=[]):
        super(RemoveFunctionModifier, self).__init__()
        self._rm_funcs = rm_funcs

    def modify(self, f, inputs):
        if f.info.type_name not in self._rm_funcs:
            return None
        return inputs[0]
