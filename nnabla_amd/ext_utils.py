"""``get_extension_context`` (mirrors python/src/nnabla/ext_utils.py:72-98)."""


def list_extensions():
    return ['hip']


def import_extension_module(ext_name):
    if ext_name != 'hip':
        raise ImportError("Extension `%s` does not exist in this build (available: hip)." % ext_name)
    from . import ext_hip
    return ext_hip


def get_extension_context(ext_name, **kw):
    return import_extension_module(ext_name).context(**kw)
