"""nnabla_amd: MI355X-native implementation of nnabla's quantization functions.

The package holds the gfx950 kernel library (``csrc/kernels`` -> ``lib/libnbla_hip_kernels.so``), the host-side C++
mirror of nnabla's Function/Array plug-in interface with the ``hip`` extension (``csrc/nbla``, ``csrc/hip`` ->
``lib/libnnabla_hip.so``) and a thin Python front-end with nnabla's names::

    import nnabla_amd as nn
    import nnabla_amd.functions as F
    from nnabla_amd.ext_utils import get_extension_context
    with nn.context_scope(get_extension_context('hip')):
        y = F.fixed_point_quantize(x)
    y.forward()

There is no CPU fallback: without the built HIP libraries every front-end call raises.
"""
__version__ = "0.1.0"

from .context import Context, context_scope, get_current_context, set_default_context  # noqa: F401
from .variable import NdArray, Variable, auto_forward, get_auto_forward, set_auto_forward  # noqa: F401
from .parameter import (clear_parameters, get_parameter, get_parameter_or_create, get_parameters,  # noqa: F401
                        parameter_scope, pop_parameter, set_parameter)
