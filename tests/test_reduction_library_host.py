"""The wave64 reduction library compiles for every element type, operator and row width the
mapper can hand it: device-only hipRTC builds for gfx950, no GPU needed.  (The reference's
library is CUB over `+` and float only, tc/core/cuda/cuda_libraries.h:214-285; values are checked
on the GPU in test_gpu_reductions.py.)"""
import pytest

import tensorcomprehensions_amd as tc

TYPES = ["int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64", "float16", "float", "double"]
# 32: lane groups inside one wavefront; 48: rows through LDS; 128: wavefront reduce + LDS partials
WIDTHS = [32, 48, 128]

ALL_OPS = """
def red({T}(N, K) I) -> (s, p, lo, hi) {{
    s(n) +=! I(n, k)
    p(n) *=! I(n, k)
    lo(n) min=! I(n, k)
    hi(n) max=! I(n, k)
}}
"""


@pytest.mark.parametrize("width", WIDTHS)
@pytest.mark.parametrize("dtype", TYPES)
def test_block_reduction_compiles_for_every_type_operator_and_width(dtype, width):
    torch_name = {"float": "float32", "double": "float64"}.get(dtype, dtype)
    ins = [tc.ShapeOnly((8, 5 * width), torch_name)]
    options = f"naive;tile=1;mapToThreads={width};mapToBlocks=8;matchLibraryCalls=1;outerScheduleFusionStrategy=Min;intraTileScheduleFusionStrategy=Min"
    ex = tc.compile(ALL_OPS.format(T=dtype), "red", ins, options)      # raises on a hipRTC error
    src = ex.compiled_source
    c_type = {"int8": "signed char", "uint8": "unsigned char", "int16": "short", "uint16": "unsigned short", "int32": "int",
              "uint32": "unsigned int", "int64": "long long", "uint64": "unsigned long long", "float16": "_Float16"}.get(dtype, dtype)
    for op in ("OpSum", "OpProd", "OpMin", "OpMax"):
        assert f"__tc::blockAllReduceX<__tc::{op}<{c_type}>, {width}, 1, 1>" in src, (op, c_type)
    assert ex.num_kernels == 4


@pytest.mark.parametrize("dtype", ["int32", "int64", "uint32", "uint64", "float", "double"])
def test_reductions_divided_among_blocks_compile_for_every_operator(dtype):
    """reductionBlocks: sums meet in an atomic add, the other operators in a compare-and-swap loop
    on the bit pattern; 32- and 64-bit element types."""
    torch_name = {"float": "float32", "double": "float64"}.get(dtype, dtype)
    ins = [tc.ShapeOnly((8, 1024), torch_name)]
    options = "naive;tile=1,1;mapToThreads=64;mapToBlocks=64,64;matchLibraryCalls=1;reductionBlocks=8"
    ex = tc.compile(ALL_OPS.format(T=dtype), "red", ins, options)      # raises on a hipRTC error
    src = ex.compiled_source
    assert ex.num_kernels == 8                                          # a fill and a sliced kernel per statement
    assert "__tc::atomicAccumulate(&ps[" in src
    for op, out in (("OpProd", "pp"), ("OpMin", "plo"), ("OpMax", "phi")):
        assert f"__tc::atomicCombine<__tc::{op}<" in src and f">>(&{out}[" in src
