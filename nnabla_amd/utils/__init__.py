"""Utilities around the function path: NNP / nntxt graph files."""
