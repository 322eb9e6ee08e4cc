"""Mapping-option sets that once broke the reference's mapper, replayed on the HIP backend: the
cases of test/cuda/test_tc_mapper_bugs.cc:112-900 (same TCs, shapes and option values; results
checked against the CPU oracle rather than against the naive mapping) and the end-to-end cases of
test/cuda/test_compile_and_run.cc:95-310 and test/cuda/test_tc_mapper.cc:47-412."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu


def opts(outer="Preserve3Coincident", intra="Max", tile=None, threads=None, blocks=None, unroll=None, shared=None,
         private=None, copy_unroll=None, library=None, fix=None):
    parts = ["naive", f"outerScheduleFusionStrategy={outer}", f"intraTileScheduleFusionStrategy={intra}"]
    for key, val in (("tile", tile), ("mapToThreads", threads), ("mapToBlocks", blocks)):
        if val is not None:
            parts.append(f"{key}=" + ",".join(map(str, val)))
    for key, val in (("unroll", unroll), ("useSharedMemory", shared), ("usePrivateMemory", private),
                     ("unrollCopyShared", copy_unroll), ("matchLibraryCalls", library),
                     ("fixParametersBeforeScheduling", fix)):
        if val is not None:
            parts.append(f"{key}={int(val)}")
    return ";".join(parts)


def check(src, entry, ins_np, options, k, scale=0.0, prefill=None):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for i, o in enumerate(outs):
        if prefill is not None:
            o.copy_(torch.from_numpy(prefill[i]))
        else:
            o.fill_(float("nan")) if o.is_floating_point() else o.fill_(-77)
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    ref = tc_oracle.run(src, entry, ins_np, outputs=[p.copy() for p in prefill] if prefill is not None else None)
    for o, r in zip(outs, ref):
        got = o.cpu().numpy()
        assert got.shape == r.shape and got.dtype == r.dtype
        if np.issubdtype(r.dtype, np.integer):
            assert np.array_equal(got, r)
        else:
            # scale: max|ref|, or the magnitude of the summed terms where the result is a cancellation
            bound = max(W.tolerance(k, r), 1e-5 * np.sqrt(k) * scale)
            assert np.abs(got.astype(np.float64) - r).max() <= bound, (entry, options, ex.launch_bounds())
    return ex


def normal(seed, *shapes):
    rng = np.random.Generator(np.random.Philox(seed))
    return [rng.standard_normal(s, dtype=np.float32) for s in shapes]


# --- test_tc_mapper_bugs.cc ----------------------------------------------------------------------
TENSORDOT_OPTIONS = {
    "BaseCorrect": "conv",
    "ReductionUnroll": opts(tile=(28, 14, 7, 32, 28, 256), blocks=(1,), threads=(7, 28), unroll=64, shared=1, private=0,
                            copy_unroll=1, library=1),
    "Reduction2": opts(tile=(28, 14, 7, 32, 9, 256), blocks=(1,), threads=(64, 10), shared=1, private=0, copy_unroll=1,
                       library=1),
    "Reduction3": opts(tile=(28, 14, 7, 32, 28, 256), blocks=(256, 256, 256), threads=(7, 32), shared=1, private=0,
                       copy_unroll=1, library=1),
    "FormerSharedIllegalAddress": opts(intra="Min", tile=(14, 4, 28, 7, 1), threads=(256,), blocks=(7, 4, 256), unroll=16,
                                       shared=1, private=1, copy_unroll=1, library=0),
    "NoUnroll": opts(intra="Min", tile=(1, 7), threads=(4, 16, 4), blocks=(14, 14, 128), unroll=256, shared=1, private=1,
                     copy_unroll=0, library=0),
    "EmptyLeaf": opts(outer="Min", intra="Min", tile=(256, 64), threads=(32,), blocks=(128, 14), unroll=8, shared=0,
                      private=0, copy_unroll=0, library=1),
    "FormerIllegalAccess": opts(intra="Preserve3Coincident", tile=(1, 7, 14), threads=(28, 16), blocks=(128, 16, 28),
                                unroll=64, shared=1, private=0, copy_unroll=1, library=0),
}


@pytest.mark.parametrize("case", sorted(TENSORDOT_OPTIONS))
def test_tensordot_32_512_8_2_28_28(case):
    print(f"tensordot {case}: {TENSORDOT_OPTIONS[case]}", flush=True)
    shapes = [(32, 512, 8, 28, 28), (32, 8, 2, 28, 28)]
    if TENSORDOT_OPTIONS[case].count("mapToBlocks=1;"):
        shapes = [(4, 64, 8, 28, 28), (4, 8, 2, 28, 28)]        # a single block: keep the run short
    check(W.TENSORDOT, "tensordot", normal(1, *shapes), TENSORDOT_OPTIONS[case], 8)


GROUP_CONV_OPTIONS = {
    "FormerSharedIllegalAddress": opts(outer="Max", intra="Min", tile=(14, 1, 1, 1, 1), threads=(14, 28), blocks=(32, 56, 1),
                                       unroll=1, shared=1, private=0, copy_unroll=1, library=0),
    "SharedPrivate": opts(outer="Max", intra="Preserve3Coincident", tile=(14, 8, 1, 64, 7, 4), threads=(32,), blocks=(8, 32),
                          unroll=1, shared=1, private=1, copy_unroll=0, library=0),
}


@pytest.mark.parametrize("case", sorted(GROUP_CONV_OPTIONS))
def test_group_convolution_32_32_4_4_56_56_3_3(case):
    print(f"group convolution {case}", flush=True)
    ins = normal(2, (32, 32, 4, 56, 56), (32, 4, 4, 3, 3), (32, 4))
    check(W.GROUP_CONVOLUTION, "group_convolution", ins, GROUP_CONV_OPTIONS[case], 36)


TMM = "def tmm(float(B, X) I, float(Y, X) W) -> (O) { O(b, y) +=! I(b, r_x) * W(y, r_x) }"


@pytest.mark.parametrize("shape,options", [
    ([(128, 1000), (1024, 1000)], opts(outer="Max", intra="Min", tile=(8, 500), threads=(125,), blocks=(128, 1000, 500), unroll=256,
                                       shared=1, private=1, copy_unroll=1, library=1)),                       # InvalidPtx
    ([(128, 1000), (1024, 1000)], opts(outer="Max", intra="Preserve3Coincident", tile=(32, 32, 250), threads=(4, 32),
                                       blocks=(63, 128), unroll=16, shared=1, private=1, copy_unroll=0, library=0)),  # IllegalAccess
    ([(128, 1024), (1024, 1024)], opts(outer="Max", intra="Max", tile=(2,), threads=(128,), blocks=(64,), unroll=16, shared=0,
                                       private=0, copy_unroll=1, library=1)),                                 # TooStrictPrecision
    ([(128, 1024), (1024, 1024)], opts(outer="Max", intra="Min", tile=(1, 1), threads=(32,), blocks=(128, 128), unroll=64,
                                       shared=1, private=1, copy_unroll=1, library=1)),                       # Tightening
    ([(128, 1024), (1000, 1024)], opts(intra="Min", tile=(1, 32, 63), threads=(2, 32), blocks=(64, 128, 1024), unroll=128,
                                       shared=0, private=0, copy_unroll=0, library=1)),                       # DisjunctiveFilter
])
def test_transposed_matmul_option_sets(shape, options):
    print(f"tmm {shape} {options}", flush=True)
    check(TMM, "tmm", normal(3, *shape), options, shape[0][1])


def test_layernorm_reference_in_two_groups():
    src = """def layernorm(float(T, B, C) I) -> (O, mean, centered, var) {
        mean(t, b) +=! I(t, b, r_c) / C
        centered(t, b, c) = I(t, b, c) - mean(t, b)
        var(t, b) +=! centered(t, b, r_c) * centered(t, b, r_c)
        var(t, b) = var(t, b) / C
        O(t, b, c) = centered(t, b, c) / rsqrt(var(t, b)) }"""
    o = opts(outer="Max", intra="Preserve3Coincident", tile=(4, 16), threads=(64,), blocks=(128, 32, 4), unroll=2, shared=1,
             private=1, copy_unroll=0, library=0)
    check(src, "layernorm", normal(4, (7, 32, 64)), o, 64)


def test_min_in_upper_bound_and_nested_subscripts():
    graph2 = """def graph2(float(N, C, H, W) I, float(N, C, R, T) J, float(KH, KW) W1) -> (O, Out) {
        O(n, c, h, w) +=! J(n, c, h + r_kh, w + r_kw) * W1(r_kh, r_kw)
        Out(c0, c1) +=! I(n, c0, h, w) * O(n, c1, h, w) }"""
    check(graph2, "graph2", normal(5, (1, 20, 40, 40), (1, 20, 42, 42), (3, 3)), "naive", 1600 * 9)
    conv = "def convolution(float(X) A, float(Xp) K) -> (B) { B(x) +=! A(xp) * K(X - 1 + x - xp) where xp in 0:X }"
    A = np.zeros(33, np.float32)
    K = np.zeros(65, np.float32)
    A[10] = 1
    K[32] = 1
    ex = check(conv, "convolution", [A, K], "naive", 33)
    (out,) = tc.prepare_outputs(conv, "convolution", [torch.from_numpy(A).cuda(), torch.from_numpy(K).cuda()])
    tc.run(ex, [torch.from_numpy(A).cuda(), torch.from_numpy(K).cuda()], [out])
    assert out[10].item() == 1.0


def test_group_norm_with_thread_mapped_reductions_terminates():
    src = """def group_norm(float(N, G, D, H, W) I, float(G, D) gamma, float(G, D) beta) -> (O, mean, var) {
        mean(n, g) +=! I(n, g, r_d, r_h, r_w)
        var(n, g) +=! I(n, g, r_d, r_h, r_w) * I(n, g, r_d, r_h, r_w)
        O(n, g, d, h, w) = gamma(g, d) * (I(n, g, d, h, w) - mean(n, g) * 1.0)
            * rsqrt(var(n, g) * 1.0 - mean(n, g) * mean(n, g) * 1.0 * 1.0 + 1e-5) + beta(g, d) }"""
    rng = np.random.Generator(np.random.Philox(6))
    I = rng.standard_normal((4, 4, 2, 6, 6), dtype=np.float32)
    I -= I.mean(axis=(2, 3, 4), keepdims=True)         # group sums ~ 0 keep the rsqrt argument positive
    o = opts(outer="Min", intra="Min", tile=(2, 6, 8, 48), unroll=4, library=1, threads=(6, 12), blocks=(8,), shared=1, private=1,
             copy_unroll=0)
    check(src, "group_norm", [I, np.ones((4, 2), np.float32), np.zeros((4, 2), np.float32)], o, 72, scale=float(np.abs(I).max()))


def test_kronecker_first_factor():
    src = "def Kronecker3_1(float(D2, N2) W2, float(M, N0, N1, N2) X) -> (XW2) { XW2(m, n0, n1, d2) +=! X(m, n0, n1, r_n2) * W2(d2, r_n2) }"
    ins = normal(7, (16, 32), (64, 32, 32, 32))
    check(src, "Kronecker3_1", ins, opts(intra="Preserve3Coincident", fix=1, tile=(256,), unroll=16, library=1, threads=(16, 8),
                                          blocks=(4, 2), shared=1, private=1, copy_unroll=1), 32)
    check(src, "Kronecker3_1", ins, opts(intra="Preserve3Coincident", fix=1, tile=(1, 32), unroll=16, library=1, threads=(32, 4),
                                          blocks=(64, 32), shared=1, private=1, copy_unroll=1), 32)


# --- test_compile_and_run.cc ---------------------------------------------------------------------
def test_softmax_variants():
    c = """def softmax(float(N, D) I) -> (O, expsum, maxVal) {
        maxVal(n) max=! I(n, d)
        expsum(n) +=! exp(I(n, d) - maxVal(n))
        O(n, d) = exp(I(n, d) - maxVal(n)) / expsum(n) }"""
    d = """def softmax(float(N, D) I) -> (O, maxVal, expDistance, expSum) {
        maxVal(n) max=! I(n, d)
        expDistance(n, d) = exp(I(n, d) - maxVal(n))
        expSum(n) +=! expDistance(n, d)
        O(n, d) = expDistance(n, d) / expSum(n) }"""
    (x,) = normal(8, (32, 16))
    for src in (c, d):
        ex = check(src, "softmax", [x], "naive", 16)
        ins = [torch.from_numpy(x).cuda()]
        outs = tc.prepare_outputs(src, "softmax", ins)
        tc.run(ex, ins, outs)
        assert torch.allclose(outs[0], torch.softmax(ins[0], 1), atol=1e-6)


def test_concat_indexing_casts_and_inplace_matmul():
    a, b = normal(9, (32, 16), (32, 16))
    check("def concat(float(M, N) A, float(M, N) B) -> (O1) { O1(n, i, m) = i == 0 ? A(m, n) : B(m, n) where i in 0:2 }",
          "concat", [a, b], "naive", 1)
    table = normal(10, (3, 4))[0]
    check("def indexing(float(H, W) input, int32(L) index) -> (output) { output(l, w) = input(index(l), w) where l in 0:2 }",
          "indexing", [table, np.array([2, 0], np.int32)], "naive", 1)
    A = (np.ones((2, 4), np.float32) / 2 + 1)
    ex = check("def cast(float(M, N) A, int32 four) -> (int32(M, N) output) { output(m, n) = int32(A(m, n) + four) }",
               "cast", [A, np.array(4, np.int32)], "naive", 1)
    assert "int* __restrict__ poutput" in ex.compiled_source
    x, y, c = normal(11, (3, 4), (4, 5), (3, 5))
    check("def matmul(float(M, N) A, float(N, K) B) -> (output) { output(m, k) += A(m, r_n) * B(r_n, k) }",
          "matmul", [x, y], "mlp", 4, prefill=[c])


@pytest.mark.parametrize("sh,sw", [(1, 1), (2, 2), (3, 2)])
def test_strided_convolution(sh, sw):
    src = f"""def convolutionStrided(float(N, C, H, W) I, float(O, C, KH, KW) W1, float(O) B) -> (O1) {{
        O1(n, o, h, w) +=! I(n, r_c, {sh} * h + r_kh, {sw} * w + r_kw) * W1(o, r_c, r_kh, r_kw)
        O1(n, o, h, w) = O1(n, o, h, w) + B(o) }}"""
    I, W1, B = normal(12, (4, 6, 20, 19), (8, 6, 3, 4), (8,))
    check(src, "convolutionStrided", [I, W1, B], "conv", 72)
    ref = torch.nn.functional.conv2d(torch.from_numpy(I), torch.from_numpy(W1), torch.from_numpy(B), stride=(sh, sw))
    ins = [torch.from_numpy(t).cuda() for t in (I, W1, B)]
    (out,) = tc.prepare_outputs(src, "convolutionStrided", ins)
    assert tuple(out.shape) == tuple(ref.shape)


@pytest.mark.parametrize("tc_type,np_type", [("uint8", np.uint8), ("int8", np.int8), ("int16", np.int16), ("int32", np.int32),
                                             ("int64", np.int64), ("float32", np.float32), ("float64", np.float64),
                                             ("float", np.float32), ("double", np.float64)])
def test_element_types(tc_type, np_type):
    src = f"def test_type({tc_type}(N) A) -> (B) {{ B(k) +=! A(i) where k in 0:1 }}"
    check(src, "test_type", [np.ones(100, np_type)], "naive", 100)


# --- test_tc_mapper.cc ---------------------------------------------------------------------------
@pytest.mark.parametrize("options", [
    "naive;tile=0;mapToBlocks=1;mapToThreads=16;matchLibraryCalls=1",
    "naive;tile=0;mapToBlocks=1;mapToThreads=16;matchLibraryCalls=1;unroll=1",
    "naive;tile=0;mapToBlocks=1;mapToThreads=16;matchLibraryCalls=1;unroll=128",
    "naive;tile=64;mapToBlocks=1;mapToThreads=64;matchLibraryCalls=1;unroll=128",
])
def test_reduction_to_a_scalar(options):
    src = "def sum1D(float(M) A) -> (C) { C(k) +=! A(r_m) where k in 0:1 }"
    check(src, "sum1D", normal(13, (1237,)), options, 1237)


def test_batch_triple_hadamard_and_matmul_schedules():
    src = "def batch_triple_hadamard(float(B, D) U, float(B, D) V, float(B, D) W) -> (Z) { Z(b, d) = U(b, d) * V(b, d) * W(b, d) }"
    check(src, "batch_triple_hadamard", normal(14, (123, 70), (123, 70), (123, 70)), "pointwise", 1)
    mm = "def matmul(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"
    for o in ("naive;tile=1,1,1;mapToBlocks=1;mapToThreads=1", "naive;tile=4,4,4;mapToBlocks=1;mapToThreads=4,4",
              "naive;tile=1,1,1;mapToThreads=4,1,1;mapToBlocks=1", "mlp"):
        check(mm, "matmul", normal(15, (17, 23), (23, 31)), o, 23)
