"""Chainable mapping options for the HIP backend.

Python face of tc::HipMappingOptions; setter names are the reference's
(tc/core/mapping_options.h:307-365, tc/core/cuda/cuda_mapping_options.h:145-245), camelCase kept
so tuned option sets read the same in both languages.  The object is a thin builder over the
library's option text; validation and defaults live in the library.
"""
import ctypes

from . import _capi


class FusionStrategy:
    Max = "Max"
    Preserve3Coincident = "Preserve3Coincident"
    Min = "Min"


def _b(v):
    return "1" if v else "0"


class MappingOptions:
    PRESETS = ("naive", "single_thread", "pointwise", "mlp", "conv", "group_conv", "unmapped")

    def __init__(self, text="naive"):
        self._parts = [p for p in str(text).split(";") if p]

    # presets (makeNaiveMappingOptions & co.)
    @classmethod
    def naive(cls): return cls("naive")
    @classmethod
    def single_thread(cls): return cls("single_thread")
    @classmethod
    def pointwise(cls): return cls("pointwise")
    @classmethod
    def mlp(cls): return cls("mlp")
    @classmethod
    def conv(cls): return cls("conv")
    @classmethod
    def group_conv(cls): return cls("group_conv")

    def _set(self, key, value):
        self._parts = [p for p in self._parts if not p.startswith(key + "=")] + [f"{key}={value}"]
        return self

    @staticmethod
    def _csv(values):
        if len(values) == 1 and isinstance(values[0], (list, tuple)):
            values = values[0]
        return ",".join(str(int(v)) for v in values)

    def tile(self, *sizes): return self._set("tile", self._csv(sizes))
    def unroll(self, n): return self._set("unroll", int(n))
    def mapToThreads(self, *sizes): return self._set("mapToThreads", self._csv(sizes))
    def mapToBlocks(self, *sizes): return self._set("mapToBlocks", self._csv(sizes))
    def scheduleFusionStrategy(self, s): return self._set("scheduleFusionStrategy", s)
    def outerScheduleFusionStrategy(self, s): return self._set("outerScheduleFusionStrategy", s)
    def intraTileScheduleFusionStrategy(self, s): return self._set("intraTileScheduleFusionStrategy", s)
    def outerScheduleAllowSkewing(self, b): return self._set("outerScheduleAllowSkewing", _b(b))
    def outerSchedulePositiveOrthant(self, b): return self._set("outerSchedulePositiveOrthant", _b(b))
    def intraTileScheduleAllowSkewing(self, b): return self._set("intraTileScheduleAllowSkewing", _b(b))
    def intraTileSchedulePositiveOrthant(self, b): return self._set("intraTileSchedulePositiveOrthant", _b(b))
    def fixParametersBeforeScheduling(self, b): return self._set("fixParametersBeforeScheduling", _b(b))
    def tileImperfectlyNested(self, b): return self._set("tileImperfectlyNested", _b(b))
    def matchLibraryCalls(self, b): return self._set("matchLibraryCalls", _b(b))
    def useSharedMemory(self, b): return self._set("useSharedMemory", _b(b))
    def usePrivateMemory(self, b): return self._set("usePrivateMemory", _b(b))
    def unrollCopyShared(self, b): return self._set("unrollCopyShared", _b(b))
    def maxSharedMemory(self, n): return self._set("maxSharedMemory", int(n))
    def useReadOnlyCache(self, b): return self._set("useReadOnlyCache", _b(b))
    def privateDepth(self, n): return self._set("privateDepth", int(n))
    def sharedDepth(self, n): return self._set("sharedDepth", int(n))
    # CDNA4 extras
    def vectorWidth(self, n): return self._set("vectorWidth", int(n))
    def collapseContiguous(self, b): return self._set("collapseContiguous", _b(b))
    def useMfma(self, b): return self._set("useMfma", _b(b))
    def prefetchShared(self, b): return self._set("prefetchShared", _b(b))
    def reductionBlocks(self, n): return self._set("reductionBlocks", int(n))

    def to_text(self):
        return ";".join(self._parts)

    def normalized(self):
        """Every field spelled out, as the library sees it."""
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().tc_options_normalize(self.to_text().encode(), ctypes.byref(out)))
        return _capi.take_string(out)

    def serialize(self):
        """toProtobufSerializedString(): proto2 wire bytes."""
        buf = ctypes.c_void_p()
        n = ctypes.c_size_t(0)
        _capi.check(_capi.lib().tc_options_to_serialized(self.to_text().encode(), ctypes.byref(buf), ctypes.byref(n)))
        data = ctypes.string_at(buf.value, n.value)
        _capi.lib().tc_free(buf)
        return data

    @classmethod
    def deserialize(cls, data):
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().tc_options_from_serialized(data, len(data), ctypes.byref(out)))
        return cls(_capi.take_string(out))

    def to_cpp(self):
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().tc_options_to_cpp(self.to_text().encode(), ctypes.byref(out)))
        return _capi.take_string(out)

    def __str__(self):
        return self.to_text()

    def __repr__(self):
        return f"MappingOptions({self.to_text()!r})"

    def __eq__(self, other):
        return isinstance(other, MappingOptions) and self.normalized() == other.normalized()
