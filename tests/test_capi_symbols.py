"""The shared libraries load on a GPU-less host and export every symbol the headers declare."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tensorcomprehensions_amd")


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tc_[a-z_0-9]+|tchip_[a-z_0-9]+)\s*\(", text)))


def test_tchip_exports():
    lib = ctypes.CDLL(os.path.join(PKG, "libtchip.so"))
    names = declared("tchip.h")
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n


def test_tc_hip_exports():
    ctypes.CDLL(os.path.join(PKG, "libtchip.so"), mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(os.path.join(PKG, "libtc_hip.so"))
    names = declared("tc_hip.h")
    assert "tc_compile" in names and "tc_autotune" in names and "tc_executor_profile" in names
    for n in names:
        assert hasattr(lib, n), n


def test_errors_do_not_cross_the_abi_as_exceptions():
    import tensorcomprehensions_amd as tc
    from tensorcomprehensions_amd import _capi
    out = ctypes.c_void_p()
    status = _capi.lib().tc_lang_dump(b"def broken(", b"function", ctypes.byref(out))
    assert status != 0
    assert b"expected" in _capi.lib().tc_last_error()
