"""Utilities around the function path: NNP / nntxt graph files (``nnp_graph``, ``nnp_format``, ``save``) and
quantization-aware training (``qnn``)."""
