"""The ``hip`` extension module: what ``nnabla_ext.<ext>`` modules provide (doc/python/api/ext.rst:30-50,
python/src/nnabla_ext/cpu/__init__.py:17-45) for the MI355X backend."""
import ctypes

from . import _capi
from .context import Context


def array_classes():
    buf = ctypes.create_string_buffer(256)
    _capi.lib().nblac_array_classes(b"hip", buf, 256)
    return buf.value.decode().split(",")


def context(device_id='0', type_config='float', **kw):
    """``Context(['hip:float', 'cpu:float'], 'HipCachedArray', device_id)``.  Functions without a hip implementation
    resolve to the next backend in the list, which in this build has no implementations and therefore raises."""
    if type_config == 'float':
        backends = ['hip:float', 'cpu:float']
    elif type_config == 'half':
        backends = ['hip:half', 'hip:float', 'cpu:float']
    else:
        raise ValueError("Unknown data type config is given %s" % type_config)
    return Context(backends, array_classes()[0], str(device_id))


def device_synchronize(device_id='0'):
    _capi.check(_capi.lib().nblac_hip_device_synchronize(str(device_id).encode()))


def synchronize(device_id='0', **kw):
    device_synchronize(device_id)


def get_device_count():
    return _capi.lib().nblac_hip_device_count()


def get_devices():
    return [str(i) for i in range(get_device_count())]


def clear_memory_cache():
    _capi.check(_capi.lib().nblac_hip_clear_memory_cache())


def allocated_bytes(device_id='0', caching=True):
    """Bytes the backend's allocator currently holds from the device."""
    return int(_capi.lib().nblac_allocator_bytes(b"hip", str(device_id).encode(), int(caching)))
