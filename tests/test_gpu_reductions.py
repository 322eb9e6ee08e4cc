"""Wave64 reduction library on the block shapes of the reference's reduction tests
(test/cuda/test_tc_mapper.cc:120-177: x extents {1,2,4,7,8,11,15,17,24,32,35,42,64,128,130} and the
(x,y) pairs), extended with whole-wavefront multiples, against the oracle and A.sum(1)."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu

SUM2D = "def sum2d(float(M, N) A) -> (C) { C(m) +=! A(m, r_n) }"
X_ONLY = [1, 2, 4, 7, 8, 11, 15, 17, 24, 32, 35, 42, 64, 128, 130, 192, 256, 320, 512, 1024]
XY = [(4, 7), (11, 5), (16, 9), (8, 11), (11, 8), (111, 7), (128, 7), (7, 128), (64, 4), (256, 4), (192, 3)]


def check(src, entry, ins_np, options, k):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    ref = tc_oracle.run(src, entry, ins_np)
    for o, r in zip(outs, ref):
        assert np.abs(o.cpu().numpy() - r).max() <= W.tolerance(k, r)
    return ex


@pytest.mark.parametrize("bx", X_ONLY)
def test_row_sums_block_x(bx):
    print(f"sum2d block x={bx}", flush=True)
    A = np.random.Generator(np.random.Philox(bx)).standard_normal((37, 1013), dtype=np.float32)
    ex = check(SUM2D, "sum2d", [A], f"naive;matchLibraryCalls=1;mapToThreads={bx};mapToBlocks=64;tile=1", 1013)
    assert ("blockAllReduceX" in ex.compiled_source) == (bx > 1)


@pytest.mark.parametrize("bx,by", XY)
def test_row_sums_block_xy(bx, by):
    print(f"sum2d block x={bx} y={by}", flush=True)
    A = np.random.Generator(np.random.Philox(bx * 1000 + by)).standard_normal((53, 700), dtype=np.float32)
    check(SUM2D, "sum2d", [A], f"naive;matchLibraryCalls=1;mapToThreads={bx},{by};mapToBlocks=16;tile={by}", 700)


def test_all_ones_sum_is_exactly_the_reduction_length():
    A = np.ones((64, 4096), np.float32)
    ins = [torch.from_numpy(A).cuda()]
    ex = tc.compile(SUM2D, "sum2d", ins, "naive;matchLibraryCalls=1;mapToThreads=256;mapToBlocks=64;tile=1;vectorWidth=4")
    (out,) = tc.prepare_outputs(SUM2D, "sum2d", ins)
    tc.run(ex, ins, [out])
    assert torch.all(out == 4096.0)


@pytest.mark.parametrize("op,ref", [("max=!", lambda a: a.max(1)), ("min=!", lambda a: a.min(1))])
def test_min_max_reductions_are_bit_exact(op, ref):
    src = f"def red(float(M, N) A) -> (C) {{ C(m) {op} A(m, r_n) }}"
    A = np.random.Generator(np.random.Philox(3)).standard_normal((40, 999), dtype=np.float32)
    ins = [torch.from_numpy(A).cuda()]
    ex = tc.compile(src, "red", ins, "naive;matchLibraryCalls=1;mapToThreads=192,2;mapToBlocks=20;tile=2")
    (out,) = tc.prepare_outputs(src, "red", ins)
    tc.run(ex, ins, [out])
    assert np.array_equal(out.cpu().numpy(), ref(A))


def test_non_initialising_reduction_accumulates_into_existing_values():
    src = "def acc(float(M, N) A) -> (C) { C(m) += A(m, r_n) }"
    A = np.ones((16, 300), np.float32)
    ins = [torch.from_numpy(A).cuda()]
    for opts in ("naive", "naive;matchLibraryCalls=1;mapToThreads=64,2;tile=2"):
        ex = tc.compile(src, "acc", ins, opts)
        out = torch.full((16,), 5.0, device="cuda")
        tc.run(ex, ins, [out])
        assert torch.all(out == 305.0), opts


def test_moments_full_size_properties():
    """Size-independent checks at the benchmark size: a row of constants has that mean and zero
    variance; shifting a row shifts the mean and keeps the variance."""
    name = "c5_moments"
    src, entry, shapes, _, k = W.CONFIGS[name]
    X = W.make_inputs(name)[0]
    X[0, :] = 2.5
    X[1, :] = X[2, :] + 10.0
    ins = [torch.from_numpy(X).cuda()]
    ex = tc.compile(src, entry, ins, W.TUNED[name])
    mean, var = tc.prepare_outputs(src, entry, ins)
    tc.run(ex, ins, [mean, var])
    mean, var = mean.cpu().numpy(), var.cpu().numpy()
    assert mean[0] == 2.5 and var[0] == 0.0
    assert abs(mean[1] - (mean[2] + 10.0)) <= 1e-4
    assert abs(var[1] - var[2]) <= 1e-3 * var[2]
    Xd = X.astype(np.float64)
    assert np.abs(mean - Xd.mean(1)).max() <= W.tolerance(k, Xd.mean(1))
    assert np.abs(var - Xd.var(1)).max() <= W.tolerance(k, Xd.var(1))


@pytest.mark.parametrize("threads,fragment", [(64, "__builtin_amdgcn_wave_barrier();"), (256, "__syncthreads();"), (32, "wave_barrier")])
def test_moments_second_stage_sees_the_mean_across_threads(threads, fragment):
    """The variance stage reads the mean that lane 0 stored: ordering inside one wavefront when
    the block is a single wavefront, a block barrier otherwise."""
    X = np.random.Generator(np.random.Philox(threads)).standard_normal((48, 2000), dtype=np.float32) + 3.0
    ex = check(W.MOMENTS, "moments", [X], f"naive;tile=1;mapToBlocks=48;matchLibraryCalls=1;mapToThreads={threads}", 2000)
    src = ex.compiled_source
    assert fragment in src[src.index("// stage 0: mean"):src.index("// stage 1: var")]


def test_point_wise_chain_needs_no_barrier():
    chain = """def f(float(N, M) A) -> (O, P) {
        O(i, j) = A(i, j) + 1.0
        P(i, j) = O(i, j) * 2.0 }"""
    A = np.random.Generator(np.random.Philox(77)).standard_normal((70, 130), dtype=np.float32)
    ex = check(chain, "f", [A], "naive", 1)
    assert "__syncthreads" not in ex.compiled_source and ex.num_kernels == 1


@pytest.mark.parametrize("threads,block", [("512,2", (64, 2, 1)), ("33,2", (33, 2, 1)), ("40,2", (33, 2, 1))])
def test_many_unrolled_reductions_on_odd_rows(threads, block):
    """17 block reductions unrolled back to back on rows of 33 threads: with one-hot columns every
    row sum is exactly 1, so a partial that goes missing or counts twice shows by position.  A row
    width the option leaves room for is widened to whole lane groups (33 -> 64)."""
    src = "def f(float(N, N) A) -> (O) { O(i) +=! fmax(A(i, j), 0) }"
    A = torch.zeros(33, 33, device="cuda")
    ex = tc.compile(src, "f", [A], f"naive;tile=64,0,2;mapToThreads={threads};mapToBlocks=64;unroll=128;matchLibraryCalls=1")
    assert ex.launch_bounds() == ((1, 1, 1), block)
    (out,) = tc.prepare_outputs(src, "f", [A])
    for c in range(33):
        A.zero_()
        A[:, c] = 1
        out.fill_(float("nan"))
        tc.run(ex, [A], [out])
        assert torch.all(out == 1.0), (c, out.cpu().numpy())


SOFTMAX = """
def softmax(float(N, D) I) -> (O, maxVal, expSum) {
    maxVal(n) max=! I(n, d)
    expSum(n) +=! exp(I(n, d) - maxVal(n))
    O(n, d) = exp(I(n, d) - maxVal(n)) / expSum(n)
}
"""


@pytest.mark.parametrize("d,threads,reads", [(1024, 64, 1), (1024, 256, 1), (1000, 64, 1), (777, 128, 1), (777, 1024, 1)])
def test_softmax_row_stays_in_registers_between_the_stages(d, threads, reads):
    """Two reductions and a pointwise stage over the same row in one kernel take it from one read
    (register cache), also where the threads over-cover the row and fold the surplus points:
    the three stages fold alike."""
    print(f"softmax d={d} threads={threads}", flush=True)
    A = np.random.Generator(np.random.Philox(d)).standard_normal((37, d), dtype=np.float32)
    ex = check(SOFTMAX, "softmax", [A], f"naive;tile=1;mapToThreads={threads};mapToBlocks=64;matchLibraryCalls=1;"
               f"vectorWidth=4;unroll=64;usePrivateMemory=1;outerScheduleFusionStrategy=Max", d)
    assert ex.num_kernels == 1 and ex.compiled_source.count("pI[") == reads


ROW_NORMALISE = """
def f(float(N, M) A) -> (S, T) {
    S(n, m) = A(n, m) + 2
    T(n) +=! A(n, m) * A(n, m)
    S(n, m) = S(n, m) / (T(n) + 1)
}
"""


@pytest.mark.parametrize("options", [
    "naive;tile=1;mapToThreads=128;mapToBlocks=64;outerScheduleFusionStrategy=Max",
    "naive;tile=1;mapToThreads=128;mapToBlocks=64;outerScheduleFusionStrategy=Max;matchLibraryCalls=1;vectorWidth=4;usePrivateMemory=1",
    "naive;tile=2,64;mapToThreads=32,2;mapToBlocks=8;outerScheduleFusionStrategy=Max;unroll=4",
    "naive;outerScheduleFusionStrategy=Min",
])
def test_tensor_rewritten_by_a_later_stage_of_the_same_kernel(options):
    """S is written, a reduction over the same rows follows, then S is rewritten from itself and
    the reduction's result: one kernel under maximal fusion (the rewrite waits behind a barrier
    for the reduction), three kernels under minimal fusion; same values."""
    A = np.random.Generator(np.random.Philox(9)).standard_normal((50, 384), dtype=np.float32)
    ex = check(ROW_NORMALISE, "f", [A], options, 384)
    assert ex.num_kernels == (3 if "Min" in options else 1)
