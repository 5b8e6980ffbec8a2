"""Graph converters (the part of python/src/nnabla/experimental/graph_converters that quantization-aware training
uses): the converter driver, the identity copy, function removal, and the two quantization modifiers."""
from .graph_converter import FunctionModifier, GraphConverter  # noqa: F401
from .identity import IdentityModifier  # noqa: F401
from .remove_function import RemoveFunctionModifier  # noqa: F401
from .quantize import QuantizeNonQNNToRecordingModifier, QuantizeRecordingToTrainingModifier  # noqa: F401
