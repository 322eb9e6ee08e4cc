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


# ------------------------------------------------------------------------------------------------
# products through the block reduction (the reference's library matches `+` only,
# tc/core/polyhedral/cuda/mapped_scop.cc:253-311): lane-group, whole-wavefront and LDS row widths
# ------------------------------------------------------------------------------------------------
PROD_WIDTHS = [(32, 32), (64, 64), (128, 128), (192, 192), (48, 48), (33, 33), (7, 7)]


def run_one(src, entry, ins_np, options, prefill=None):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for i, o in enumerate(outs):
        if prefill is not None:
            o.copy_(torch.from_numpy(prefill[i]))
        elif o.dtype.is_floating_point:
            o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs], ex


@pytest.mark.parametrize("threads,block_x", PROD_WIDTHS)
def test_row_products_near_one(threads, block_x):
    """Factors 1 + N(0, 0.01): the product stays finite and its relative error is bounded like a
    sum's (log of the product = sum of the logs)."""
    src = "def prod(float(M, N) A) -> (C) { C(m) *=! A(m, r_n) }"
    A = (1.0 + 0.01 * np.random.Generator(np.random.Philox(threads)).standard_normal((29, 1000))).astype(np.float32)
    (got,), ex = run_one(src, "prod", [A], f"naive;matchLibraryCalls=1;mapToThreads={threads};mapToBlocks=29;tile=1")
    assert ex.launch_bounds()[1][0] == block_x
    assert "blockAllReduceX<__tc::OpProd<float>" in ex.compiled_source
    (ref,) = tc_oracle.run(src, "prod", [A])
    exact = A.astype(np.float64).prod(1)
    assert np.abs(ref - exact).max() <= 1e-5 * np.sqrt(1000) * np.abs(exact).max()      # the oracle itself
    assert np.abs(got - ref).max() <= W.tolerance(1000, ref)


@pytest.mark.parametrize("threads,block_x", PROD_WIDTHS)
def test_row_products_of_small_integers_are_exact(threads, block_x):
    """Signs and at most twenty factors of two per row: every partial product is an exact fp32
    value whatever the order, so the result is bit for bit the oracle's and the closed form."""
    src = "def prod(float(M, N) A) -> (C) { C(m) *=! A(m, r_n) }"
    rng = np.random.Generator(np.random.Philox(1000 + threads))
    A = rng.choice(np.array([1.0, -1.0], np.float32), size=(31, 777))
    twos = np.zeros(31, np.int64)
    for m in range(31):
        cols = rng.choice(777, size=int(rng.integers(0, 21)), replace=False)
        A[m, cols] *= 2.0
        twos[m] = len(cols)
    (got,), _ = run_one(src, "prod", [A], f"naive;matchLibraryCalls=1;mapToThreads={threads};mapToBlocks=16;tile=1")
    closed = np.where((A < 0).sum(1) % 2 == 1, -1.0, 1.0) * 2.0 ** twos
    (ref,) = tc_oracle.run(src, "prod", [A])
    assert np.array_equal(ref, closed.astype(np.float32))
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("threads", [32, 128, 48])
def test_non_initialising_product_multiplies_into_existing_values(threads):
    src = "def prod(float(M, N) A) -> (C) { C(m) *= A(m, r_n) }"
    A = np.full((8, 300), 1.0, np.float32)
    A[:, ::100] = 2.0                                   # three factors of two per row
    prior = np.arange(1, 9, dtype=np.float32)
    (got,), _ = run_one(src, "prod", [A], f"naive;matchLibraryCalls=1;mapToThreads={threads};mapToBlocks=8;tile=1",
                        prefill=[prior.copy()])
    assert np.array_equal(got, prior * 8.0)


# ------------------------------------------------------------------------------------------------
# unsigned and boolean tensors on the device (test/cuda/test_compile_and_run.cc:259-310 runs
# uint8, the signed integers and the floats; the other unsigned widths and bool complete the set)
# ------------------------------------------------------------------------------------------------
UNSIGNED = [("uint8", np.uint8), ("uint16", np.uint16), ("uint32", np.uint32), ("uint64", np.uint64)]


def device_tensor(array):
    """torch has no arithmetic for the wider unsigned types, but it can hold their bits."""
    return torch.from_numpy(array).cuda()


@pytest.mark.parametrize("tc_type,np_type", UNSIGNED)
@pytest.mark.parametrize("threads", [1, 32, 48, 128])
def test_unsigned_reductions_match_the_oracle_bit_for_bit(tc_type, np_type, threads):
    src = f"""
def red({tc_type}(M, N) A) -> (s, lo, hi) {{
    s(m) +=! A(m, r_n)
    lo(m) min=! A(m, r_n)
    hi(m) max=! A(m, r_n)
}}
"""
    info = np.iinfo(np_type)
    rng = np.random.Generator(np.random.Philox(7))
    # values in the upper half of the range tell unsigned comparisons from signed ones; the sums wrap
    A = rng.integers(info.max // 2, info.max, size=(9, 500), dtype=np_type, endpoint=True)
    A[:, 3] = rng.integers(0, 5, size=9).astype(np_type)
    lib = "matchLibraryCalls=1;" if threads > 1 else ""
    got, ex = run_one(src, "red", [A], f"naive;{lib}mapToThreads={max(threads, 1)};mapToBlocks=9;tile=1")
    ref = tc_oracle.run(src, "red", [A])
    for g, r, name in zip(got, ref, ("sum", "min", "max")):
        assert g.dtype == r.dtype == np.dtype(np_type), name
        assert np.array_equal(g, r), name
    assert np.array_equal(ref[0], A.sum(1, dtype=np_type))           # wrap-around sum
    assert np.array_equal(ref[1], A.min(1)) and np.array_equal(ref[2], A.max(1))


@pytest.mark.parametrize("tc_type,np_type", UNSIGNED)
def test_unsigned_pointwise_arithmetic(tc_type, np_type):
    src = f"def f({tc_type}(N) A, {tc_type}(N) B) -> (C, D) {{ C(i) = A(i) / B(i) + A(i) % B(i)\n D(i) = max(A(i), B(i)) - min(A(i), B(i)) }}"
    info = np.iinfo(np_type)
    rng = np.random.Generator(np.random.Philox(8))
    A = rng.integers(info.max // 2, info.max, size=1000, dtype=np_type, endpoint=True)
    B = rng.integers(1, 1000 if info.max > 1000 else info.max, size=1000, dtype=np_type)
    got, _ = run_one(src, "f", [A, B], "naive")
    ref = tc_oracle.run(src, "f", [A, B])
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and np.array_equal(g, r)
    assert np.array_equal(ref[0].astype(np_type), (A // B + A % B).astype(np_type))
    assert np.array_equal(ref[1].astype(np_type), np.maximum(A, B) - np.minimum(A, B))


def test_bool_tensors_on_the_device():
    src = """
def f(bool(M, N) P, float(M, N) X) -> (cnt, sel, any) {
    cnt(m) +=! P(m, r_n) ? 1 : 0
    sel(m, n) = P(m, n) ? X(m, n) : 0.0
    any(m) max=! P(m, r_n) ? 1 : 0
}
"""
    rng = np.random.Generator(np.random.Philox(9))
    P = rng.random((12, 130)) > 0.7
    P[5] = False
    X = rng.standard_normal((12, 130), dtype=np.float32)
    for options in ("naive", "naive;matchLibraryCalls=1;mapToThreads=64;mapToBlocks=12;tile=1,0"):
        got, _ = run_one(src, "f", [P, X], options)
        ref = tc_oracle.run(src, "f", [P, X])
        for g, r in zip(got, ref):
            assert np.array_equal(g, r), options
        assert np.array_equal(ref[0], P.sum(1).astype(ref[0].dtype))
        assert np.array_equal(ref[1], np.where(P, X, np.float32(0)))
        assert np.array_equal(ref[2], P.any(1).astype(ref[2].dtype))
