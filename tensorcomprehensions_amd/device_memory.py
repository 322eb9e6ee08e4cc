"""Device memory without a tensor library: a dense row-major array in HIP device memory that
the entry points of this package accept wherever they accept a torch tensor.

For hosts that have no PyTorch, or that must not load it (PyTorch brings its own copy of the
HIP runtime and of hipRTC; a process that holds DeviceBuffers only uses the ROCm installation's).
Allocation and copies go through the thin HIP layer libtchip.so (include/tchip.h); numpy carries
the data on the host side.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_hip = None


def _tchip():
    global _hip
    if _hip is None:
        path = os.path.join(_HERE, "libtchip.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')} libs`")
        _hip = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        _hip.tchip_malloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        _hip.tchip_free_device.argtypes = [ctypes.c_void_p]
        _hip.tchip_memcpy_to_device.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        _hip.tchip_memcpy_to_host.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        _hip.tchip_last_error_string.restype = ctypes.c_char_p
        _hip.tchip_get_device.argtypes = [ctypes.POINTER(ctypes.c_int)]
        _hip.tchip_device_name.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    return _hip


def _check(status, what):
    if status != 0:
        raise RuntimeError(f"{what} failed: {_tchip().tchip_last_error_string().decode('utf-8', 'replace')}")


def device_name(device=None):
    """Name of the (current) HIP device."""
    hip = _tchip()
    if device is None:
        cur = ctypes.c_int(0)
        _check(hip.tchip_get_device(ctypes.byref(cur)), "hipGetDevice")
        device = cur.value
    buf = ctypes.create_string_buffer(256)
    _check(hip.tchip_device_name(device, buf, 256), "device name query")
    return buf.value.decode()


class DeviceBuffer:
    """`shape` elements of `dtype` (a numpy dtype or its name) on the current HIP device,
    uninitialised; freed when the object goes away."""

    is_cuda = True

    def __init__(self, shape, dtype="float32"):
        hip = _tchip()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        cur = ctypes.c_int(0)
        _check(hip.tchip_get_device(ctypes.byref(cur)), "hipGetDevice")
        self.device_index = cur.value
        self._ptr = ctypes.c_void_p()
        _check(hip.tchip_malloc(ctypes.byref(self._ptr), max(self.nbytes, 1)), "hipMalloc")

    def __del__(self):
        ptr, self._ptr = getattr(self, "_ptr", None), None
        if ptr and _hip is not None:
            _hip.tchip_free_device(ptr)

    @classmethod
    def from_numpy(cls, array):
        array = np.ascontiguousarray(array)
        buf = cls(array.shape, array.dtype)
        _check(_tchip().tchip_memcpy_to_device(buf._ptr, array.ctypes.data_as(ctypes.c_void_p), buf.nbytes),
               "copy to the device")
        return buf

    def numpy(self):
        """A host copy (synchronises with the device)."""
        out = np.empty(self.shape, dtype=self.dtype)
        _check(_tchip().tchip_memcpy_to_host(out.ctypes.data_as(ctypes.c_void_p), self._ptr, self.nbytes),
               "copy to the host")
        return out

    def data_ptr(self):
        return self._ptr.value or 0

    @property
    def dtype_name(self):
        return "bool" if self.dtype == np.bool_ else self.dtype.name

    def stride(self):
        strides, acc = [], 1
        for s in reversed(self.shape):
            strides.insert(0, acc)
            acc *= s
        return tuple(strides)

    def numel(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def element_size(self):
        return self.dtype.itemsize
