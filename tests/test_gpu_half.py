"""float16 tensors (accepted here; the reference's front end stops at the type, tc/lang/sema.h:62-66,
and its own type sweep leaves it out, test/test_tc2halide.cc:201-222).  Arithmetic is IEEE half,
rounded after every operation, on the device as in the oracle (which compiles such nests with
clang, `-fexcess-precision=16`).  Inputs are chosen so that every intermediate is exactly
representable; one case with arbitrary values allows the fused multiply-adds of the device code
their one rounding less."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle

pytestmark = pytest.mark.gpu

HALF = """
def h(float16(M, N) X, float16(N) w, float16(M, N) Y) -> (s, mx, mn, z, f, p) {
    s(m) +=! X(m, n) * w(n)
    mx(m) max=! X(m, n)
    mn(m) min=! Y(m, n)
    z(m, n) = X(m, n) * Y(m, n) + w(n)
    f(m) +=! float(X(m, n)) * float(Y(m, n))
    p(m) *=! (X(m, n) == 0 ? w(n) * 0 + 1 : w(n) * 0 + 1)
}
"""
OPTIONS = [
    "naive",
    "naive;tile=1,64;mapToThreads=64;mapToBlocks=256;matchLibraryCalls=1;unroll=4",
    "naive;tile=2,128;mapToThreads=32,2;mapToBlocks=64;matchLibraryCalls=1;vectorWidth=4;unroll=8",
    "naive;tile=4,32;mapToThreads=32,4;mapToBlocks=64,64;useSharedMemory=1;unroll=4;useReadOnlyCache=1",
    "naive;tile=1,0;mapToThreads=256;mapToBlocks=64;matchLibraryCalls=1;outerScheduleFusionStrategy=Max;usePrivateMemory=1",
]


def run(src, entry, ins_np, options):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs], ex


@pytest.mark.parametrize("options", OPTIONS)
def test_half_arithmetic_and_reductions_exact(options):
    rng = np.random.Generator(np.random.Philox(16))
    X = rng.integers(-3, 4, size=(37, 300)).astype(np.float16)
    w = rng.integers(-2, 3, size=300).astype(np.float16)
    Y = rng.integers(-3, 4, size=(37, 300)).astype(np.float16)
    ref = tc_oracle.run(HALF, "h", [X, w, Y])
    assert [r.dtype for r in ref] == [np.float16, np.float16, np.float16, np.float16, np.float32, np.float16]
    Xf, wf, Yf = X.astype(np.float32), w.astype(np.float32), Y.astype(np.float32)
    # the oracle on closed forms: every partial sum stays below 2048 in magnitude, exact in half
    assert np.array_equal(ref[0], (Xf @ wf).astype(np.float16)) and np.abs(Xf * wf).sum(1).max() < 2048
    assert np.array_equal(ref[1], X.max(1)) and np.array_equal(ref[2], Y.min(1))
    assert np.array_equal(ref[3], (Xf * Yf + wf).astype(np.float16))
    assert np.array_equal(ref[4], (Xf * Yf).sum(1)) and np.all(ref[5] == 1)
    got, ex = run(HALF, "h", [X, w, Y], options)
    assert "_Float16" in ex.compiled_source
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and np.array_equal(g, r), options


def test_half_with_arbitrary_values_within_one_rounding():
    src = "def f(float16(N) a, float16(N) b, float16(N) c) -> (o, e) { o(i) = a(i) * b(i) + c(i)\n e(i) = exp(a(i)) }"
    rng = np.random.Generator(np.random.Philox(17))
    a, b, c = [rng.standard_normal(5000).astype(np.float16) for _ in range(3)]
    (o, e), _ = run(src, "f", [a, b, c], "naive;mapToThreads=256;vectorWidth=2")
    ro, re_ = tc_oracle.run(src, "f", [a, b, c])
    exact = a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)
    prod = np.abs(a.astype(np.float64) * b.astype(np.float64))
    ulp = (np.maximum(np.abs(exact), 2.0 ** -14) + prod) * 2.0 ** -10      # a rounding of the product, one of the sum
    assert np.all(np.abs(ro.astype(np.float64) - exact) <= ulp)        # two roundings
    assert np.all(np.abs(o.astype(np.float64) - exact) <= ulp)         # one (fused) or two
    assert re_.dtype == e.dtype
    assert np.all(np.abs(e.astype(np.float64) - re_.astype(np.float64)) <= np.abs(re_.astype(np.float64)) * 2.0 ** -9)
