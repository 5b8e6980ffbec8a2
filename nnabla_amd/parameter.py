"""Parameter scopes (the subset of python/src/nnabla/parameter.py the parametric functions need): a tree of ordered
dictionaries addressed with '/'-separated names, ``parameter_scope`` to descend, ``get_parameter_or_create`` to
register."""
from collections import OrderedDict
from contextlib import contextmanager

import numpy as np

from .variable import Variable

current_scope = OrderedDict()
root_scope = current_scope


@contextmanager
def parameter_scope(name, scope=None):
    """``with parameter_scope('conv1'):`` -- parameters created inside are registered under ``conv1/``."""
    global current_scope
    names = name.strip('/').split('/')
    if not names or not names[0]:
        raise ValueError('Invalid argument of parameter_scope("{}").'.format(name))
    prev = current_scope
    cur = current_scope if scope is None else scope
    for n in names:
        nxt = cur.get(n)
        if nxt is None:
            nxt = OrderedDict()
            cur[n] = nxt
        elif not isinstance(nxt, dict):
            raise ValueError("%r is a parameter, not a scope." % n)
        cur = nxt
    current_scope = cur
    try:
        yield current_scope
    finally:
        current_scope = prev


def _split(name):
    names = name.split('/')
    return names[:-1], names[-1]


def get_parameter(key):
    scopes, leaf = _split(key)
    cur = current_scope
    for n in scopes:
        cur = cur.get(n)
        if not isinstance(cur, dict):
            return None
    v = cur.get(leaf)
    return v if isinstance(v, Variable) else None


def set_parameter(key, param):
    scopes, leaf = _split(key)
    if scopes:
        with parameter_scope('/'.join(scopes)):
            return set_parameter(leaf, param)
    current_scope[leaf] = param


def pop_parameter(key):
    scopes, leaf = _split(key)
    cur = current_scope
    for n in scopes:
        cur = cur.get(n)
        if not isinstance(cur, dict):
            return None
    return cur.pop(leaf, None)


def get_parameter_or_create(name, shape=None, initializer=None, need_grad=True, as_need_grad=None):
    """The parameter registered under ``name`` in the current scope, created from ``initializer`` (a callable
    shape -> array, or an array) when it does not exist yet.  ``as_need_grad``: the ``need_grad`` of the returned
    variable when it should differ from the registered one (an unlinked view is returned then)."""
    scopes, leaf = _split(name)
    if scopes:
        with parameter_scope('/'.join(scopes)):
            return get_parameter_or_create(leaf, shape, initializer, need_grad, as_need_grad)
    param = get_parameter(name)
    if param is None:
        if isinstance(initializer, np.ndarray):
            if shape is not None and tuple(shape) != initializer.shape:
                raise ValueError("The initializer's shape %s differs from the requested %s."
                                 % (initializer.shape, tuple(shape)))
            param = Variable.from_numpy_array(initializer.astype(np.float32), need_grad=need_grad)
        else:
            if initializer is None or shape is None:
                raise ValueError("A shape and an initializer are needed to create parameter %r." % name)
            param = Variable.from_numpy_array(np.asarray(initializer(shape=tuple(shape)), np.float32),
                                              need_grad=need_grad)
        param.name = name
        set_parameter(name, param)
    else:
        if shape is not None and tuple(param.shape) != tuple(shape):
            raise ValueError("Parameter %r exists with shape %s, requested %s."
                             % (name, tuple(param.shape), tuple(shape)))
    if as_need_grad is None or param.need_grad == as_need_grad:
        return param
    return param.get_unlinked_variable(need_grad=as_need_grad)


def get_parameters(params=None, path='', grad_only=True):
    """Flat ordered dictionary 'scope/name' -> variable of the current scope (those with need_grad by default)."""
    if params is None:
        params = OrderedDict()
    for k, v in current_scope.items():
        if isinstance(v, dict):
            with parameter_scope(k):
                get_parameters(params, path + '/' + k if path else k, grad_only)
        else:
            if grad_only and not v.need_grad:
                continue
            params[path + '/' + k if path else k] = v
    return params


def clear_parameters():
    current_scope.clear()
