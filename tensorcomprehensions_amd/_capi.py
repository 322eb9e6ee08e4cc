"""ctypes binding of libtc_hip.so (the C ABI declared in include/tc_hip.h).

Loading fails loudly when the library has not been built: there is no fallback path.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtc_hip.so")
TC_MAX_RANK = 8


class DLContext(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("ctx", DLContext),
        ("ndim", ctypes.c_int32),
        ("dtype", DLDataType),
        ("shape", ctypes.POINTER(ctypes.c_int64)),
        ("strides", ctypes.POINTER(ctypes.c_int64)),
        ("byte_offset", ctypes.c_uint64),
    ]


class TensorInfo(ctypes.Structure):
    _fields_ = [
        ("dtype", DLDataType),
        ("ndim", ctypes.c_int32),
        ("shape", ctypes.c_int64 * TC_MAX_RANK),
        ("strides", ctypes.c_int64 * TC_MAX_RANK),
    ]


class TcError(RuntimeError):
    """A C++ exception caught at the C ABI (lang::ErrorReport text, TC_CHECK failure, HIP error)."""


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')} libs` "
                "(or python -c 'import __graft_entry__ as g; g.build()')")
        _lib = ctypes.CDLL(_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        _declare(_lib)
    return _lib


def _declare(l):
    P = ctypes.POINTER
    tensors = P(P(DLTensor))
    l.tc_last_error.restype = ctypes.c_char_p
    l.tc_free.argtypes = [ctypes.c_void_p]
    l.tc_free.restype = None
    l.tc_set_compiler_options.argtypes = [ctypes.c_int, ctypes.c_int]
    l.tc_set_compiler_options.restype = None
    l.tc_infer_output_info.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int,
                                       P(TensorInfo), ctypes.c_int, P(ctypes.c_int)]
    l.tc_compile.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int, ctypes.c_char_p,
                             P(ctypes.c_void_p)]
    l.tc_compile_serialized_options.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int,
                                                ctypes.c_void_p, ctypes.c_size_t, P(ctypes.c_void_p)]
    l.tc_executor_run.argtypes = [ctypes.c_void_p, tensors, ctypes.c_int, tensors, ctypes.c_int, ctypes.c_void_p]
    l.tc_executor_unchecked_run.argtypes = [ctypes.c_void_p, P(ctypes.c_void_p), ctypes.c_int,
                                            P(ctypes.c_void_p), ctypes.c_int, ctypes.c_void_p]
    l.tc_executor_profile.argtypes = [ctypes.c_void_p, tensors, ctypes.c_int, tensors, ctypes.c_int,
                                      ctypes.c_void_p, P(ctypes.c_double), P(ctypes.c_double)]
    l.tc_executor_profile_repeated.argtypes = [ctypes.c_void_p, P(ctypes.c_void_p), ctypes.c_int,
                                               P(ctypes.c_void_p), ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                                               P(ctypes.c_double)]
    l.tc_executor_source.argtypes = [ctypes.c_void_p]
    l.tc_executor_source.restype = ctypes.c_char_p
    l.tc_executor_num_kernels.argtypes = [ctypes.c_void_p]
    l.tc_executor_launch_bounds.argtypes = [ctypes.c_void_p, ctypes.c_int, P(ctypes.c_uint), P(ctypes.c_uint)]
    l.tc_executor_kernel_name.argtypes = [ctypes.c_void_p, ctypes.c_int]
    l.tc_executor_kernel_name.restype = ctypes.c_char_p
    l.tc_executor_lds_bytes.argtypes = [ctypes.c_void_p, ctypes.c_int]
    l.tc_executor_lds_bytes.restype = ctypes.c_int64
    l.tc_executor_clear.argtypes = [ctypes.c_void_p]
    l.tc_executor_destroy.argtypes = [ctypes.c_void_p]
    l.tc_executor_destroy.restype = None
    l.tc_options_normalize.argtypes = [ctypes.c_char_p, P(ctypes.c_void_p)]
    l.tc_options_to_serialized.argtypes = [ctypes.c_char_p, P(ctypes.c_void_p), P(ctypes.c_size_t)]
    l.tc_options_from_serialized.argtypes = [ctypes.c_void_p, ctypes.c_size_t, P(ctypes.c_void_p)]
    l.tc_options_to_cpp.argtypes = [ctypes.c_char_p, P(ctypes.c_void_p)]
    l.tc_map.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int, ctypes.c_char_p,
                         P(ctypes.c_void_p), P(ctypes.c_int), P(ctypes.c_uint), P(ctypes.c_uint)]
    l.tc_lang_dump.argtypes = [ctypes.c_char_p, ctypes.c_char_p, P(ctypes.c_void_p)]
    l.tc_host_query.argtypes = [ctypes.c_char_p, ctypes.c_char_p, P(ctypes.c_void_p)]
    l.tc_autotune.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int, tensors, ctypes.c_int,
                              ctypes.c_char_p, ctypes.c_char_p, P(ctypes.c_void_p)]
    l.tc_options_cache_load.argtypes = [ctypes.c_char_p, ctypes.c_char_p, tensors, ctypes.c_int, ctypes.c_char_p,
                                        ctypes.c_int, P(ctypes.c_void_p)]


def check(status):
    if status != 0:
        raise TcError(lib().tc_last_error().decode("utf-8", "replace"))


def take_string(ptr):
    """Copy and free a malloc'ed C string returned through a char** parameter."""
    s = ctypes.string_at(ptr.value).decode("utf-8", "replace")
    lib().tc_free(ptr)
    return s


# dtype code/bits per numpy/torch dtype name
DTYPES = {
    "float16": (2, 16), "float32": (2, 32), "float64": (2, 64), "int8": (0, 8), "int16": (0, 16), "int32": (0, 32),
    "int64": (0, 64), "uint8": (1, 8), "uint16": (1, 16), "uint32": (1, 32), "uint64": (1, 64), "bool": (1, 8),
}


class TensorPack:
    """Keeps the ctypes DLTensor structs (and their shape/stride arrays) of a tensor list alive."""

    def __init__(self, metas):
        # metas: iterable of (data_ptr, dtype_name, shape, strides, device_type, device_id)
        self.items = []
        self.keep = []
        for ptr, dtype, shape, strides, dev_type, dev_id in metas:
            n = len(shape)
            sh = (ctypes.c_int64 * max(n, 1))(*shape)
            st = (ctypes.c_int64 * max(n, 1))(*strides)
            code, bits = DTYPES[dtype]
            t = DLTensor(ctypes.c_void_p(ptr), DLContext(dev_type, dev_id), n, DLDataType(code, bits, 1),
                         ctypes.cast(sh, ctypes.POINTER(ctypes.c_int64)),
                         ctypes.cast(st, ctypes.POINTER(ctypes.c_int64)), 0)
            self.keep.append((sh, st))
            self.items.append(t)
        self.array = (ctypes.POINTER(DLTensor) * max(len(self.items), 1))(
            *[ctypes.pointer(t) for t in self.items])

    @property
    def ptr(self):
        return ctypes.cast(self.array, ctypes.POINTER(ctypes.POINTER(DLTensor)))

    def __len__(self):
        return len(self.items)
