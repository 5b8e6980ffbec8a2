"""Experimental utilities mirrored from ``nnabla.experimental``: the graph converters used by quantization-aware
training."""
