"""Loader of libtc_hip_testing.so: host-side test scaffolding (a synthetic genetic search, the
tuning loop on a cost model, a sample options cache) that is built next to the product library
and kept out of it."""
import ctypes
import os

from tensorcomprehensions_amd import _capi

_PATH = os.path.join(os.path.dirname(os.path.abspath(_capi.__file__)), "libtc_hip_testing.so")
_lib = None


def scaffold_query(what, arg=""):
    global _lib
    if _lib is None:
        _capi.lib()                                   # the product library first (shared symbols)
        if not os.path.exists(_PATH):
            raise ImportError(f"{_PATH} is missing: build it with `make -C tensorcomprehensions_amd/csrc libs`")
        _lib = ctypes.CDLL(_PATH, mode=ctypes.RTLD_GLOBAL)
        _lib.tc_testing_query.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    out = ctypes.c_void_p()
    _capi.check(_lib.tc_testing_query(what.encode(), str(arg).encode(), ctypes.byref(out)))
    return _capi.take_string(out)
