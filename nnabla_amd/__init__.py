"""nnabla_amd: MI355X-native implementation of nnabla's quantization functions.

The package holds the gfx950 kernel library (``csrc/kernels`` -> ``lib/``), the
host-side C++ mirror of nnabla's Function/Array plug-in interface (``csrc/nbla``,
``csrc/hip``) and thin Python front-ends.  There is no CPU fallback: importing a
front-end without the built HIP libraries raises.
"""
__version__ = "0.1.0"
