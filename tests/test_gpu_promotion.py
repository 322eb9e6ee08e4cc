"""LDS promotion beyond the reduction operands of one stage, against the oracle: a footprint two
stages of a kernel share, a stage without a reduction (overlapping windows), copies whose last
block-wide step is ragged or whose loops overshoot."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W
from tests.test_mapper import STENCIL, TWO_CONVOLUTIONS

pytestmark = pytest.mark.gpu


def run(src, entry, ins_np, options):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs], ex


@pytest.mark.parametrize("options", [
    "naive;tile=1,8,10,10;mapToThreads=10,10;mapToBlocks=4;unroll=8;useSharedMemory=1;outerScheduleFusionStrategy=Max",
    "naive;tile=2,4,5,10;mapToThreads=10,5;mapToBlocks=2,2,2;unroll=8;useSharedMemory=1;outerScheduleFusionStrategy=Max",
    "naive;tile=1,8,10,10;mapToThreads=10,10;mapToBlocks=2;unroll=8;useSharedMemory=1;outerScheduleFusionStrategy=Max",   # kernel-level loop over n
    "naive;tile=1,8,0,0;mapToThreads=64,4;mapToBlocks=4;useMfma=1;useSharedMemory=1;outerScheduleFusionStrategy=Max",
])
def test_two_convolutions_over_one_staged_input(options):
    rng = np.random.Generator(np.random.Philox(41))
    ins = [rng.integers(-3, 4, size=s).astype(np.float32) for s in [(4, 3, 12, 12), (8, 3, 3, 3), (8, 3, 3, 3)]]
    got, ex = run(TWO_CONVOLUTIONS, "two", ins, options)
    ref = tc_oracle.run(TWO_CONVOLUTIONS, "two", ins)
    torch_ref = [torch.nn.functional.conv2d(torch.from_numpy(ins[0]), torch.from_numpy(w)).numpy() for w in ins[1:]]
    for g, r, t in zip(got, ref, torch_ref):
        assert np.array_equal(r, t)                       # small integers: exact whatever the order
        assert np.array_equal(g, r), (options, ex.launch_bounds())


@pytest.mark.parametrize("options", [
    "naive;tile=8,64;mapToThreads=64,2;mapToBlocks=16,16;unroll=4;useSharedMemory=1",
    "naive;tile=8,64;mapToThreads=64,2;mapToBlocks=3,2;unroll=4;useSharedMemory=1",          # blocks loop over tiles
    "naive;tile=16,32;mapToThreads=32,4;mapToBlocks=16,16;unroll=8;useSharedMemory=1;vectorWidth=2",
    "naive;tile=5,7;mapToThreads=7,5;mapToBlocks=32,32;unroll=1;useSharedMemory=1",
    "naive;tile=16,32;mapToThreads=32,4;mapToBlocks=16,16;unroll=1;useSharedMemory=1",        # per-thread loop stays a loop
    "naive;tile=16,64;mapToThreads=16,2;mapToBlocks=2,2;unroll=2;useSharedMemory=1",          # and under block-level tile loops
])
def test_stencil_through_lds(options):
    A = np.random.Generator(np.random.Philox(42)).standard_normal((100, 200), dtype=np.float32)
    (got,), ex = run(STENCIL, "blur", [A], options)
    (ref,) = tc_oracle.run(STENCIL, "blur", [A])
    assert "lds0_A" in ex.compiled_source, options
    assert got.shape == (99, 198)
    assert np.abs(got - ref).max() <= W.tolerance(6, ref)
    closed = (A[:-1, :-2] + A[:-1, 1:-1] + A[:-1, 2:] + A[1:, :-2] + A[1:, 1:-1] + A[1:, 2:]) / 6.0
    assert np.abs(ref - closed).max() <= W.tolerance(6, ref)


@pytest.mark.parametrize("threads,shapes", [((19, 2), [(5, 26, 40), (5, 40, 19)]), ((32, 3), [(3, 33, 48), (3, 48, 37)]),
                                            ((64, 1), [(2, 70, 25), (2, 25, 90)])])
def test_staging_copies_whose_loops_overshoot_the_footprint(threads, shapes):
    """A chunked copy loop runs more iterations than the footprint needs, and the last needed one
    is ragged: nothing may be written past the LDS array (batched matmul, whole batch per block)."""
    rng = np.random.Generator(np.random.Philox(43))
    ins = [rng.integers(-3, 4, size=s).astype(np.float32) for s in shapes]
    options = f"naive;tile=64,5;mapToThreads={threads[0]},{threads[1]};mapToBlocks=16;unroll=64;useSharedMemory=1;vectorWidth=4"
    got, ex = run(W.BATCH_MATMUL, "batch_matmul", ins, options)
    (ref,) = tc_oracle.run(W.BATCH_MATMUL, "batch_matmul", ins)
    assert ex.lds_bytes() > 0
    assert np.array_equal(got[0], ref) and np.array_equal(ref, np.matmul(ins[0], ins[1]))


@pytest.mark.parametrize("options", [
    "naive;tile=32,32;mapToThreads=16,16;mapToBlocks=8,8;unroll=1;useSharedMemory=1",
    "naive;tile=32,32,0;mapToThreads=16,8;mapToBlocks=2,2;unroll=2;useSharedMemory=1",
    "naive;tile=8,64;mapToThreads=32,2;mapToBlocks=16,4;unroll=4;useSharedMemory=1;usePrivateMemory=1",
])
def test_matmul_staged_ahead_of_per_thread_loops(options):
    """A register tile that is not fully unrolled: the block tile's operands are staged once, in
    front of the per-thread loops."""
    rng = np.random.Generator(np.random.Philox(44))
    A = rng.integers(-3, 4, size=(100, 72)).astype(np.float32)
    B = rng.integers(-3, 4, size=(72, 130)).astype(np.float32)
    src = "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, k) * B(k, n) }"
    (got,), ex = run(src, "mm", [A, B], options)
    assert "lds0_A" in ex.compiled_source or "lds0_B" in ex.compiled_source, options
    assert np.array_equal(got, A @ B)


@pytest.mark.parametrize("options", [
    "naive;tile=32,32;mapToThreads=32,8;mapToBlocks=128,128;unroll=4;useSharedMemory=1",
    "naive;tile=64,64;mapToThreads=64,4;mapToBlocks=3,5;unroll=16;useSharedMemory=1",
    "naive;tile=16,24;mapToThreads=24,4;mapToBlocks=64,64;unroll=1;useSharedMemory=1",
])
def test_transposed_read_is_staged_for_coalescing(options):
    """No element is used twice, but the threads of a wavefront walk the slow dimension of A: the
    copy reads whole rows instead (the reference's promotionImprovesCoalescing rule)."""
    src = "def tr(float(N, M) A) -> (O) { O(j, i) = A(i, j) }"
    A = np.random.Generator(np.random.Philox(45)).standard_normal((300, 500), dtype=np.float32)
    (got,), ex = run(src, "tr", [A], options)
    assert "lds0_A" in ex.compiled_source
    assert np.array_equal(got, A.T)
    (ref,) = tc_oracle.run(src, "tr", [A])
    assert np.array_equal(got, ref)


CHAIN = """def chain(float(M, K) A, float(K, N) W) -> (B, C, D) {
    B(m, k) = A(m, k) * 2.0 + 1.0
    C(m, n) +=! B(m, r_k) * W(r_k, n)
    D(m) +=! C(m, r_n) + B(m, 0)
}"""


@pytest.mark.parametrize("options,forwarded", [
    ("naive;tile=4,32;mapToThreads=32,4;mapToBlocks=64;useSharedMemory=1;outerScheduleFusionStrategy=Max;unroll=4", True),
    # blocks loop over row tiles: the copies in LDS are rewritten every iteration
    ("naive;tile=4,32;mapToThreads=32,4;mapToBlocks=3;useSharedMemory=1;outerScheduleFusionStrategy=Max;unroll=4", True),
    ("naive;tile=8,16;mapToThreads=64,2;mapToBlocks=5;useSharedMemory=1;outerScheduleFusionStrategy=Max;useMfma=1", True),
    ("naive;tile=4,32;mapToThreads=32,4;mapToBlocks=64;useSharedMemory=0;outerScheduleFusionStrategy=Max;unroll=4", False),
    # a budget the producer's box does not fit: the readers go to memory
    ("naive;tile=4,32;mapToThreads=32,4;mapToBlocks=64;useSharedMemory=1;maxSharedMemory=512;outerScheduleFusionStrategy=Max", False),
])
def test_producer_to_consumer_through_lds(options, forwarded):
    """A tensor one stage of a kernel writes and later stages read is kept in LDS as well for the
    block's part of it: the readers never go to memory for it."""
    rng = np.random.Generator(np.random.Philox(46))
    A = rng.integers(-3, 4, size=(40, 48)).astype(np.float32)
    Wt = rng.integers(-3, 4, size=(48, 70)).astype(np.float32)
    got, ex = run(CHAIN, "chain", [A, Wt], options)
    assert ("fwd0_B[" in ex.compiled_source) == forwarded, options
    B = A * 2 + 1
    C = B @ Wt
    D = C.sum(1) + 70 * B[:, 0]
    ref = tc_oracle.run(CHAIN, "chain", [A, Wt])
    for r, closed in zip(ref, (B, C, D)):
        assert np.array_equal(r, closed)                   # small integers: exact in any order
    for g, r in zip(got, ref):
        assert np.array_equal(g, r), options


SOFTMAX = """def softmax(float(M, N) X) -> (mx, s, Y) {
    mx(m) max=! X(m, n)
    s(m) +=! exp(X(m, n) - mx(m))
    Y(m, n) = exp(X(m, n) - mx(m)) / s(m) }"""


@pytest.mark.parametrize("shape,options", [
    ((37, 1000), "naive;tile=1;mapToThreads=128;mapToBlocks=64;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max"),
    # blocks that loop over the rows; a row length no thread count divides
    ((37, 777), "naive;tile=1;mapToThreads=256;mapToBlocks=8;matchLibraryCalls=1;usePrivateMemory=1;vectorWidth=4;outerScheduleFusionStrategy=Max"),
    ((5, 4096), "naive;tile=1,0;mapToThreads=512;mapToBlocks=256;matchLibraryCalls=1;usePrivateMemory=1;unroll=64;vectorWidth=2;outerScheduleFusionStrategy=Max"),
    # a row of threads that is no multiple of the wavefront
    ((19, 300), "naive;tile=1;mapToThreads=100;mapToBlocks=4;matchLibraryCalls=1;usePrivateMemory=1;useSharedMemory=1;outerScheduleFusionStrategy=Max"),
    # rows of the tensor along threadIdx.y: a wavefront per row, two rows per wavefront, two wavefronts per row
    ((37, 1000), "naive;tile=4;mapToThreads=64,4;mapToBlocks=64;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max"),
    ((37, 300), "naive;tile=8;mapToThreads=32,8;mapToBlocks=3;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max"),
    ((9, 2048), "naive;tile=2;mapToThreads=128,2;mapToBlocks=64;matchLibraryCalls=1;usePrivateMemory=1;vectorWidth=4;outerScheduleFusionStrategy=Max"),
])
def test_reduction_results_forwarded_in_registers(shape, options):
    """The maximum and the sum of a row are handed to the later stages in a register: same values
    as through memory (the oracle's order for the maximum, the tolerance of a sum for the rest),
    and the stored per-row results are those the later stages used."""
    X = np.random.Generator(np.random.Philox(48)).standard_normal(shape).astype(np.float32) * 3
    got, ex = run(SOFTMAX, "softmax", [X], options)
    assert "rfwd0_mx" in ex.compiled_source and "rfwd1_s" in ex.compiled_source and ex.num_kernels == 1
    ref = tc_oracle.run(SOFTMAX, "softmax", [X])
    assert np.array_equal(got[0], ref[0])                          # a maximum has no rounding
    np.testing.assert_allclose(got[1], ref[1], rtol=1e-5 * np.sqrt(shape[1]))
    np.testing.assert_allclose(got[2], ref[2], rtol=1e-5 * np.sqrt(shape[1]), atol=1e-12)
    # the forwarded values are the stored ones: recomputing the last stage from them is exact up to exp's rounding
    np.testing.assert_allclose(got[2], np.exp(X - got[0][:, None]) / got[1][:, None], rtol=2e-6, atol=1e-12)
    np.testing.assert_allclose(got[2].sum(1), 1.0, rtol=1e-5 * np.sqrt(shape[1]))


LOG_SUM_EXP = """def lse(float(N, K) I) -> (m, e, O) {
    m(n) max=! I(n, r_k)
    m(n) = m(n) * 0.5
    e(n) +=! exp(I(n, r_k) - m(n))
    e(n) = log(e(n)) + m(n)
    O(n, k) = I(n, k) - e(n) }"""

GROUP_MOMENTS = """def gm(float(N, G, K) I) -> (s, q) {
    s(n, g) +=! I(n, g, r_k)
    q(n, g) +=! I(n, g, r_k) * I(n, g, r_k)
    s(n, g) = s(n, g) / K
    q(n, g) = q(n, g) / K - s(n, g) * s(n, g) }"""


@pytest.mark.parametrize("src,entry,shape,options,registers", [
    # updates in the epilogue of the reductions, then a reader over the whole row
    (LOG_SUM_EXP, "lse", (13, 700),
     "naive;tile=1;mapToThreads=128;mapToBlocks=64;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max", ("rfwd0_m", "rfwd1_e")),
    (LOG_SUM_EXP, "lse", (13, 700),
     "naive;tile=2,0;mapToThreads=64,2;mapToBlocks=3;matchLibraryCalls=1;usePrivateMemory=1;vectorWidth=4;outerScheduleFusionStrategy=Max", ("rfwd0_m", "rfwd1_e")),
    # updates as stages of their own behind both reductions (tc/benchmarks/moments.h:52-59 over two indices)
    (GROUP_MOMENTS, "gm", (6, 5, 333),
     "naive;tile=1,1,0;mapToThreads=100;mapToBlocks=256,256;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max", ("rfwd0_s", "rfwd1_q")),
    (GROUP_MOMENTS, "gm", (3, 2, 4096),
     "naive;tile=1,1,0;mapToThreads=256;mapToBlocks=2,2;matchLibraryCalls=1;usePrivateMemory=1;vectorWidth=4;unroll=16;useReadOnlyCache=1;outerScheduleFusionStrategy=Max",
     ("rfwd0_s", "rfwd1_q")),
])
def test_in_place_updates_of_forwarded_reductions(src, entry, shape, options, registers):
    """A reduction's result that later statements update in place stays in the register of the
    threads that hold it; the stored values are those of the last update."""
    X = np.random.Generator(np.random.Philox(49)).standard_normal(shape).astype(np.float32) * 2
    got, ex = run(src, entry, [X], options)
    assert all(r in ex.compiled_source for r in registers) and ex.num_kernels == 1
    ref = tc_oracle.run(src, entry, [X])
    k = shape[-1]
    for g, r in zip(got, ref):
        np.testing.assert_allclose(g, r, rtol=1e-5 * np.sqrt(k), atol=1e-5 * np.sqrt(k))
    if entry == "gm":
        np.testing.assert_allclose(got[0], X.mean(2), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(got[1], X.var(2), rtol=1e-4, atol=1e-5)
    else:
        half_max = X.max(1) * 0.5
        assert np.array_equal(got[0], half_max.astype(np.float32))
        lse = np.log(np.exp(X.astype(np.float64)).sum(1))
        np.testing.assert_allclose(got[1], lse, rtol=1e-5)
        np.testing.assert_allclose(got[2], X - got[1][:, None], rtol=1e-6, atol=1e-6)   # the reader saw the stored value


def test_reader_of_other_blocks_rows_stays_in_a_kernel_of_its_own():
    """Rows another block produces are read through memory, after the producing kernel: such a
    reader is not fused with its producer, and nothing is forwarded."""
    src = """def shifted(float(M, K) A) -> (B, C) {
        B(m, k) = A(m, k) + 1.0
        C(m, k) = B(m + 1, k) + B(m, k) where m in 0:M-1
    }"""
    A = np.random.Generator(np.random.Philox(47)).integers(-9, 10, size=(33, 40)).astype(np.float32)
    opts = "naive;tile=4,40;mapToThreads=40,4;mapToBlocks=64;useSharedMemory=1;outerScheduleFusionStrategy=Max"
    got, ex = run(src, "shifted", [A], opts)
    assert "fwd0_B" not in ex.compiled_source and ex.num_kernels == 2
    ref = tc_oracle.run(src, "shifted", [A])
    assert np.array_equal(ref[1], (A[1:] + 1) + (A[:-1] + 1))
    for g, r in zip(got, ref):
        assert np.array_equal(g, r)


@pytest.mark.parametrize("sub,shape", [("2 * i + 1", (42, 420)), ("5 * i", (42, 420)), ("3 * i + 2", (70, 200))])
@pytest.mark.parametrize("options", [
    "naive;tile=32,32;mapToThreads=32,8;mapToBlocks=64,64;useSharedMemory=1;unroll=4",
    "naive;tile=16,64;mapToThreads=64,4;mapToBlocks=2,2;useSharedMemory=1;unroll=1",
])
def test_strided_footprints(sub, shape, options):
    """Only the elements the computation touches are staged (test_cuda_mapper_memory_promotion.cc:709-751)."""
    src = "def strided(float(N, M) I) -> (O) { O(i, j) = I(j, %s) }" % sub
    I = np.random.Generator(np.random.Philox(48)).standard_normal(shape, dtype=np.float32)
    (got,), ex = run(src, "strided", [I], options)
    assert "lds0_I" in ex.compiled_source
    (ref,) = tc_oracle.run(src, "strided", [I])
    a, b = [int(x) for x in sub.replace("* i", "").replace("+", " ").split()] if "+" in sub else (int(sub.split()[0]), 0)
    n = (shape[1] - 1 - b) // a + 1
    assert np.array_equal(ref, I[:, b:b + a * (n - 1) + 1:a].T)
    assert np.array_equal(got, ref)


def test_strided_convolution_keeps_every_element():
    # 2 * w + k with k in 0..4 touches every column: nothing to leave out
    src = "def sconv(float(N, W) I, float(K) F) -> (O) { O(n, w) +=! I(n, 2 * w + k) * F(k) }"
    rng = np.random.Generator(np.random.Philox(49))
    I = rng.integers(-3, 4, size=(30, 131)).astype(np.float32)
    F = rng.integers(-3, 4, size=(5,)).astype(np.float32)
    (got,), ex = run(src, "sconv", [I, F], "naive;tile=4,32;mapToThreads=32,4;mapToBlocks=64,64;useSharedMemory=1;unroll=4")
    assert "lds0_I" in ex.compiled_source and " / 2]" not in ex.compiled_source
    (ref,) = tc_oracle.run(src, "sconv", [I, F])
    closed = sum(I[:, k:k + 2 * 63 + 1:2] * F[k] for k in range(5))
    assert np.array_equal(ref, closed) and np.array_equal(got, ref)
