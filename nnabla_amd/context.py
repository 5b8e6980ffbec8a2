"""Execution contexts (mirrors python/src/nnabla/context.py and the Context of _init.pyx)."""
from contextlib import contextmanager


class Context(object):
    """backend list (tried in order per function), array class, device id."""

    def __init__(self, backend=None, array_class='', device_id='0'):
        if backend is None:
            backend = ['cpu:float']
        if isinstance(backend, str):
            backend = [backend]
        self.backend = list(backend)
        self.array_class = array_class
        self.device_id = str(device_id)

    def __repr__(self):
        return "Context(backend=%r, array_class=%r, device_id=%r)" % (self.backend, self.array_class, self.device_id)

    def __eq__(self, other):
        return (isinstance(other, Context) and self.backend == other.backend and
                self.array_class == other.array_class and self.device_id == other.device_id)


_current_ctx = Context(['cpu:float'], 'CpuCachedArray', '0')


def get_current_context():
    return _current_ctx


def set_default_context(ctx):
    global _current_ctx
    _current_ctx = ctx


@contextmanager
def context_scope(ctx):
    """``with context_scope(ctx):`` functions created inside use ``ctx`` (context.py:28-50)."""
    global _current_ctx
    prev = _current_ctx
    _current_ctx = ctx
    try:
        yield ctx
    finally:
        _current_ctx = prev
