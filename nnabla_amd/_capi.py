"""ctypes loader of the host library (``lib/libnnabla_hip.so``: nbla core + hip extension + C API).

The library links the kernel library; there is no Python-side compute and no CPU fallback.  A missing library, or
any C++ ``nbla::Exception``, surfaces as a Python exception of the class nnabla raises for the same error code.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnnabla_hip.so")


class NblaError(RuntimeError):
    """Base of the exceptions translated from nbla::Exception."""


class NblaValueError(NblaError, ValueError):
    pass


class NblaTypeError(NblaError, TypeError):
    pass


class NblaNotImplementedError(NblaError, NotImplementedError):
    pass


class NblaMemoryError(NblaError, MemoryError):
    pass


class NblaIOError(NblaError, IOError):
    pass


# nbla::error_code (+1) -> exception class, as python/src/nnabla/_init.pyx translates them
_ERRORS = {1: NblaError, 2: NblaNotImplementedError, 3: NblaValueError, 4: NblaTypeError, 5: NblaMemoryError,
           6: NblaIOError, 7: NblaError, 8: NblaError, 9: NblaError, 10: NblaError}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NblaError("%s is missing: build it with `make -C nnabla_amd/csrc`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        L.nblac_last_error.restype = ctypes.c_char_p
        L.nblac_variable_new.restype = ctypes.c_void_p
        L.nblac_function_create.restype = ctypes.c_void_p
        L.nblac_function_copy.restype = ctypes.c_void_p
        L.nblac_variable_device_pointer.restype = ctypes.c_void_p
        L.nblac_variable_modification_count.restype = ctypes.c_int64
        L.nblac_allocator_bytes.restype = ctypes.c_int64
        _lib = L
        check(L.nblac_init())
    return _lib


def check(rc):
    if rc != 0:
        L = _lib
        raise _ERRORS.get(rc, NblaError)(L.nblac_last_error().decode(errors="replace"))


def check_handle(h):
    if not h:
        check(_lib.nblac_last_error_code() or 1)
    return ctypes.c_void_p(h)
