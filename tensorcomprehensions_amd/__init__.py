"""tensorcomprehensions_amd — Python face of the MI355X-native Tensor Comprehensions backend.

The functions mirror the reference's ATen entry points one-to-one
(tc/aten/aten_compiler.h:35-92, tc/aten/aten_autotuner.h:44-90):

    compile(tc, entry_point, inputs, options)      -> Executor
    prepare_outputs(tc, entry_point, inputs)       -> [torch.Tensor]   (uninitialised, like the reference)
    infer_output_tensor_info(tc, entry_point, inputs)
    run(executor, inputs, outputs)                 no synchronisation
    profile(executor, inputs, outputs)             -> ProfilingInfo(cpu_overhead_us, kernel_runtime_us)
    unchecked_run(executor, inputs, outputs)       raw pointers, no metadata checks
    autotune(tc, entry_point, inputs, base_options, **settings) -> [MappingOptions]

torch is used for device memory and the current stream only; all work happens in
libtc_hip.so through its C ABI.  There is no CPU or eager fallback.
"""
from collections import namedtuple
import ctypes

from . import _capi
from ._capi import TcError
from .device_memory import DeviceBuffer, device_name
from .mapping_options import MappingOptions, FusionStrategy

__all__ = [
    "compile", "prepare_outputs", "infer_output_tensor_info", "run", "profile", "profile_repeated", "unchecked_run", "autotune",
    "map_only", "lang_dump", "host_query", "set_compiler_options", "ShapeOnly", "DeviceBuffer", "device_name", "Executor", "MappingOptions", "FusionStrategy", "ProfilingInfo", "TcError",
]

ProfilingInfo = namedtuple("ProfilingInfo", ["cpu_overhead_us", "kernel_runtime_us"])

_TORCH_NAMES = None


def _dtype_name(t):
    return str(t.dtype).replace("torch.", "")


def _metas(tensors):
    out = []
    for t in tensors:
        if isinstance(t, DeviceBuffer):
            out.append((t.data_ptr(), t.dtype_name, t.shape, t.stride(), 10, t.device_index))
            continue
        dev_type = 10 if t.is_cuda else 1           # kDLROCM / kDLCPU
        dev_id = t.device.index or 0
        out.append((t.data_ptr(), _dtype_name(t), tuple(t.shape), tuple(t.stride()), dev_type, dev_id))
    return out


class ShapeOnly:
    """Stand-in for a tensor when only metadata matters (compile-time checks on a GPU-less host)."""

    def __init__(self, shape, dtype="float32", strides=None):
        self.shape = tuple(shape)
        self.dtype_name = dtype
        if strides is None:
            strides, acc = [], 1
            for s in reversed(self.shape):
                strides.insert(0, acc)
                acc *= s
        self.strides = tuple(strides)


def _pack(tensors):
    metas = []
    plain = []
    for t in tensors:
        if isinstance(t, ShapeOnly):
            metas.append((0, t.dtype_name, t.shape, t.strides, 10, 0))
        else:
            plain.append(t)
            metas.append(None)
    it = iter(_metas(plain))
    metas = [m if m is not None else next(it) for m in metas]
    return _capi.TensorPack(metas)


def _stream():
    """PyTorch's current stream when the caller has PyTorch loaded, else the default stream.
    (PyTorch is never imported from here: a process that works on DeviceBuffers stays without it.)"""
    import sys
    torch = sys.modules.get("torch")
    if torch is not None and torch.cuda.is_available():
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(0)


class Executor:
    """A compiled, size-specialised TC (TcExecutor<HipBackend>, tc/core/tc_executor.h:67-121)."""

    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _capi is not None:                      # module globals are gone at interpreter exit
            _capi.lib().tc_executor_destroy(h)

    def __call__(self, *inputs, outputs=None, unchecked=False):
        """Run on `inputs`; allocates the outputs unless given.  Returns one tensor or a tuple, like
        the reference's Executor.__call__ (tensor_comprehensions/__init__.py:80-121)."""
        if outputs is None:
            if self._signature is None:
                raise TcError("outputs must be passed: this executor does not know its TC")
            outputs = prepare_outputs(self._signature[0], self._signature[1], list(inputs))
        outputs = list(outputs) if isinstance(outputs, (list, tuple)) else [outputs]
        (unchecked_run if unchecked else run)(self, list(inputs), outputs)
        return outputs[0] if len(outputs) == 1 else tuple(outputs)

    _signature = None

    @property
    def compiled_source(self):
        return _capi.lib().tc_executor_source(self._h).decode()

    @property
    def num_kernels(self):
        return _capi.lib().tc_executor_num_kernels(self._h)

    def launch_bounds(self, kernel=0):
        g = (ctypes.c_uint * 3)()
        b = (ctypes.c_uint * 3)()
        _capi.check(_capi.lib().tc_executor_launch_bounds(self._h, kernel, g, b))
        return tuple(g), tuple(b)

    def grid(self):
        return self.launch_bounds(0)[0]

    def block(self):
        return self.launch_bounds(0)[1]

    def kernel_name(self, kernel=0):
        return _capi.lib().tc_executor_kernel_name(self._h, kernel).decode()

    def lds_bytes(self, kernel=0):
        return _capi.lib().tc_executor_lds_bytes(self._h, kernel)

    def clear_runtime_compiled_function(self):
        _capi.check(_capi.lib().tc_executor_clear(self._h))


def _opt_text(options):
    if options is None:
        return b"naive"
    if isinstance(options, MappingOptions):
        return options.to_text().encode()
    return str(options).encode()


def infer_output_tensor_info(tc, entry_point, inputs):
    """[(dtype_name, shape, strides)] of the outputs (tc::aten::inferOutputTensorInfo)."""
    pack = _pack(inputs)
    infos = (_capi.TensorInfo * 16)()
    count = ctypes.c_int(0)
    _capi.check(_capi.lib().tc_infer_output_info(tc.encode(), entry_point.encode(), pack.ptr, len(pack),
                                                 infos, 16, ctypes.byref(count)))
    names = {v: k for k, v in _capi.DTYPES.items() if k != "bool"}
    out = []
    for i in range(count.value):
        t = infos[i]
        out.append((names[(t.dtype.code, t.dtype.bits)], tuple(t.shape[:t.ndim]), tuple(t.strides[:t.ndim])))
    return out


def prepare_outputs(tc, entry_point, inputs):
    """Allocate output tensors on the device of inputs[0] (tc::aten::prepareOutputs,
    tc/aten/aten_compiler.cc:46-67): needs at least one input; memory is uninitialised."""
    if len(inputs) == 0:
        raise TcError("NYI: Need >0 inputs to determine the backend for the outputs")
    if isinstance(inputs[0], DeviceBuffer):
        return [DeviceBuffer(shape, name) for name, shape, _ in infer_output_tensor_info(tc, entry_point, inputs)]
    import torch
    return [torch.empty(shape, dtype=getattr(torch, name), device=inputs[0].device)
            for name, shape, _ in infer_output_tensor_info(tc, entry_point, inputs)]


def compile(tc, entry_point, inputs, options=None):
    pack = _pack(inputs)
    handle = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_compile(tc.encode(), entry_point.encode(), pack.ptr, len(pack),
                                       _opt_text(options), ctypes.byref(handle)))
    ex = Executor(handle)
    ex._signature = (tc, entry_point)
    return ex


def run(executor, inputs, outputs):
    pin, pout = _pack(inputs), _pack(outputs)
    _capi.check(_capi.lib().tc_executor_run(executor._h, pin.ptr, len(pin), pout.ptr, len(pout), _stream()))
    return outputs


def unchecked_run(executor, inputs, outputs):
    ins = (ctypes.c_void_p * max(len(inputs), 1))(*[t.data_ptr() for t in inputs])
    outs = (ctypes.c_void_p * max(len(outputs), 1))(*[t.data_ptr() for t in outputs])
    _capi.check(_capi.lib().tc_executor_unchecked_run(executor._h, ins, len(inputs), outs, len(outputs), _stream()))
    return outputs


def profile(executor, inputs, outputs):
    pin, pout = _pack(inputs), _pack(outputs)
    k, c = ctypes.c_double(0), ctypes.c_double(0)
    _capi.check(_capi.lib().tc_executor_profile(executor._h, pin.ptr, len(pin), pout.ptr, len(pout), _stream(),
                                                ctypes.byref(k), ctypes.byref(c)))
    return ProfilingInfo(c.value, k.value)


def profile_repeated(executor, inputs, outputs, repeats):
    """Device time in microseconds of `repeats` back-to-back launches (one event pair around all)."""
    ins = (ctypes.c_void_p * max(len(inputs), 1))(*[t.data_ptr() for t in inputs])
    outs = (ctypes.c_void_p * max(len(outputs), 1))(*[t.data_ptr() for t in outputs])
    total = ctypes.c_double(0)
    _capi.check(_capi.lib().tc_executor_profile_repeated(executor._h, ins, len(inputs), outs, len(outputs), _stream(),
                                                         int(repeats), ctypes.byref(total)))
    return total.value


def set_compiler_options(emit_warnings=True, throw_warnings=False):
    """tc::CompilerOptions for this thread's following calls."""
    _capi.lib().tc_set_compiler_options(int(emit_warnings), int(throw_warnings))


def map_only(tc, entry_point, inputs, options=None):
    """Run the mapper without JIT: returns (hip_source, [(grid, block), ...])."""
    pack = _pack(inputs)
    src = ctypes.c_void_p()
    n = ctypes.c_int(0)
    grids = (ctypes.c_uint * 24)()
    blocks = (ctypes.c_uint * 24)()
    _capi.check(_capi.lib().tc_map(tc.encode(), entry_point.encode(), pack.ptr, len(pack), _opt_text(options),
                                   ctypes.byref(src), ctypes.byref(n), grids, blocks))
    launches = [(tuple(grids[3 * k:3 * k + 3]), tuple(blocks[3 * k:3 * k + 3])) for k in range(n.value)]
    return _capi.take_string(src), launches


def lang_dump(text, what):
    out = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_lang_dump(text.encode(), what.encode(), ctypes.byref(out)))
    return _capi.take_string(out)


def host_query(what, arg=""):
    """Device-free tuner logic (divisor sets, search space, synthetic genetic search, cache self-test)."""
    out = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_host_query(what.encode(), str(arg).encode(), ctypes.byref(out)))
    return _capi.take_string(out)


def autotune(tc, entry_point, inputs, base_options=None, outputs=None, **settings):
    """Genetic search over mapping options (ATenAutotuner<HipBackend, GeneticSearch>::tune).
    Returns the best options first.  Settings: generations, pop_size, crossover_rate,
    mutation_rate, number_elites, threads, seed, top_k, cache_file."""
    if outputs is None:
        outputs = prepare_outputs(tc, entry_point, inputs)
    pin, pout = _pack(inputs), _pack(outputs)
    text = ";".join(f"{k}={v}" for k, v in settings.items())
    best = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_autotune(tc.encode(), entry_point.encode(), pin.ptr, len(pin), pout.ptr, len(pout),
                                        _opt_text(base_options), text.encode(), ctypes.byref(best)))
    return [MappingOptions(line) for line in _capi.take_string(best).splitlines() if line]


def load_from_cache(tc, entry_point, inputs, cache_file, count=1):
    """The `count` best options a tuning run stored for this TC and these sizes in `cache_file`
    (the reference's MappingOptionsCache.load, tensor_comprehensions/__init__.py:278-296); [] when
    the file or the entry is missing."""
    pack = _pack(inputs)
    best = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_options_cache_load(tc.encode(), entry_point.encode(), pack.ptr, len(pack),
                                                  str(cache_file).encode(), int(count), ctypes.byref(best)))
    return [MappingOptions(line) for line in _capi.take_string(best).splitlines() if line]


from .highlevel import (TC, TunerConfig, assert_almost_equal, autotune_and_compile, define,  # noqa: E402
                        make_autograd, make_autotuned_options_factory, make_load_from_cache_options_factory,
                        make_naive_options_factory)
from .symbolic import SymbolicRanges, infer_ranges  # noqa: E402
