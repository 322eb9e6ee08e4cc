"""reductionBlocks: a sum whose outermost reduction index is divided among blocks that add their
partial results into the output with atomics (the reference keeps a reduction inside one block,
mapped_scop.cc:253-383).  Integer sums are exact in any order; floating-point sums are held to the
tolerance every other summation order is held to."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu

BIAS_GRAD = "def bias_grad(float(N, M, H, W) d_O) -> (d_B) { d_B(m) +=! d_O(r_n, m, r_h, r_w) }"
STATS = """def stats(float(N, C, H, W) I) -> (sum, mean, centered) {
    sum(c) +=! I(r_n, c, r_h, r_w)
    mean(c) = sum(c) / (N * H * W)
    centered(n, c, h, w) = I(n, c, h, w) - mean(c)
}"""
OPTION_SETS = [
    "naive;tile=1,1;mapToThreads=256;mapToBlocks=64,64;matchLibraryCalls=1;reductionBlocks=16",
    "naive;tile=1,16,16;mapToThreads=64,4;mapToBlocks=8,8,8;useMfma=1;reductionBlocks=4",
    "naive;tile=1,4;mapToThreads=64,4;mapToBlocks=8,4;matchLibraryCalls=1;reductionBlocks=8;unroll=4",
    "naive;tile=2,8;mapToThreads=8,16;mapToBlocks=256,256;matchLibraryCalls=0;reductionBlocks=64;vectorWidth=2",
    "naive;tile=1,32;mapToThreads=32;mapToBlocks=3;reductionBlocks=5;outerScheduleFusionStrategy=Max",
]


def run(src, entry, ins_np, options, outs_init=None):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for i, o in enumerate(outs):
        if outs_init is not None:
            o.copy_(torch.from_numpy(outs_init[i]))
        else:
            o.fill_(float("nan") if o.dtype.is_floating_point else -77)
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs], ex


@pytest.mark.parametrize("options", OPTION_SETS)
def test_bias_gradient_split_over_blocks(options):
    d_O = np.random.Generator(np.random.Philox(61)).integers(-3, 4, size=(20, 24, 9, 7)).astype(np.float32)
    (got,), ex = run(BIAS_GRAD, "bias_grad", [d_O], options)
    assert "__tc::atomicAccumulate(&pd_B[" in ex.compiled_source and ex.num_kernels == 2
    (ref,) = tc_oracle.run(BIAS_GRAD, "bias_grad", [d_O])
    assert np.array_equal(ref, d_O.sum((0, 2, 3)))
    assert np.array_equal(got, ref)                        # small integers: exact in any order
    # run it again on the same outputs: the zeroing kernel precedes the partial sums every time
    ins = [torch.from_numpy(d_O).cuda()]
    outs = [torch.from_numpy(got.copy()).cuda()]
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    assert np.array_equal(outs[0].cpu().numpy(), ref)


@pytest.mark.parametrize("options", OPTION_SETS)
def test_readers_of_a_split_sum_wait_for_all_of_it(options):
    I = np.random.Generator(np.random.Philox(62)).standard_normal((20, 6, 9, 7), dtype=np.float32)
    got, ex = run(STATS, "stats", [I], options)
    ref = tc_oracle.run(STATS, "stats", [I])
    assert ex.num_kernels >= 3
    for g, r in zip(got, ref):
        assert np.abs(g - r).max() <= W.tolerance(20 * 9 * 7, r)


@pytest.mark.parametrize("dtype,tc_type", [(np.int32, "int32"), (np.int64, "int64"), (np.uint32, "uint32"), (np.float64, "double")])
def test_accumulating_into_existing_values_and_other_types(dtype, tc_type):
    src = f"def acc({tc_type}(M, K) X) -> (s) {{ s(m) += X(m, r_k) * X(m, r_k) }}"
    X = np.random.Generator(np.random.Philox(63)).integers(0, 9, size=(33, 600)).astype(dtype)
    prior = np.arange(33).astype(dtype)
    (got,), ex = run(src, "acc", [X], "naive;tile=1,1;mapToThreads=64;mapToBlocks=64,64;matchLibraryCalls=1;reductionBlocks=8",
                     outs_init=[prior])
    assert ex.num_kernels == 1 and "atomicAccumulate" in ex.compiled_source       # "+=": nothing to zero
    assert np.array_equal(got, prior + (X.astype(np.int64) ** 2).sum(1).astype(dtype))


def test_matrix_product_divided_among_blocks_on_the_matrix_cores():
    src = "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"
    rng = np.random.Generator(np.random.Philox(64))
    A = rng.integers(-3, 4, size=(40, 640)).astype(np.float32)
    Bm = rng.integers(-3, 4, size=(640, 50)).astype(np.float32)
    opts = "naive;tile=1,16,16;mapToThreads=64,4;mapToBlocks=8,8,8;useMfma=1;reductionBlocks=8"
    (got,), ex = run(src, "mm", [A, Bm], opts)
    s = ex.compiled_source
    assert "__builtin_amdgcn_mfma_f32_16x16x4f32" in s and "__tc::atomicAccumulate(&pC[" in s and "ksplit0_" in s
    assert np.array_equal(got, A @ Bm)


def test_the_tuner_divides_a_sum_with_few_outputs():
    """From the naive options: with 64 outputs the search may divide the sum among blocks (the gene
    is searched only where outputs are few) and has a structured starting point that does."""
    d_O = torch.randn(32, 64, 56, 56, generator=torch.Generator().manual_seed(3)).cuda()
    outs = tc.prepare_outputs(BIAS_GRAD, "bias_grad", [d_O])
    best = tc.autotune(BIAS_GRAD, "bias_grad", [d_O], "naive", outputs=outs, generations=3, pop_size=30, threads=16, seed=5, top_k=1)
    ex = tc.compile(BIAS_GRAD, "bias_grad", [d_O], best[0])
    tc.run(ex, [d_O], outs)
    torch.cuda.synchronize()
    ref = d_O.double().sum((0, 2, 3)).float()
    assert (outs[0] - ref).abs().max().item() <= W.tolerance(32 * 56 * 56, ref.cpu().numpy())

    def time_of(e):
        tc.profile_repeated(e, [d_O], outs, 50)
        return min(tc.profile_repeated(e, [d_O], outs, 20) for _ in range(5))
    plain = tc.compile(BIAS_GRAD, "bias_grad", [d_O],
                       "naive;tile=1;mapToThreads=1024;mapToBlocks=64;matchLibraryCalls=1;vectorWidth=4;useReadOnlyCache=1")
    # 64 blocks cannot fill 256 compute units: whatever the search settles on beats the best
    # mapping that keeps each sum inside one block (25.8 us against about 10)
    assert time_of(ex) < time_of(plain), best[0].to_text()


@pytest.mark.parametrize("dtype,tc_type", [(np.float32, "float"), (np.float64, "double"), (np.int32, "int32"),
                                           (np.int64, "int64"), (np.uint32, "uint32"), (np.uint64, "uint64")])
def test_minimum_maximum_and_product_divided_among_blocks(dtype, tc_type):
    src = f"""def red({tc_type}(M, K) X) -> (lo, hi, p, cnt) {{
        lo(m) min=! X(m, k)
        hi(m) max=! X(m, k)
        p(m) *=! ((X(m, k) > 5) ? 2 : 1)
        cnt(m) +=! ((X(m, k) > 5) ? 1 : 0)
    }}"""
    X = np.random.Generator(np.random.Philox(65)).integers(0, 200, size=(19, 1200)).astype(dtype)
    X[3] = 150                                       # a row without any small value
    X[:, ::40] = 7                                   # about thirty factors of two per row
    if np.issubdtype(dtype, np.signedinteger) or np.issubdtype(dtype, np.floating):
        X[5] = -X[5] - 1                             # an all-negative row: the maximum must not start at zero
    got, ex = run(src, "red", [X], "naive;tile=1,1;mapToThreads=64;mapToBlocks=64,64;matchLibraryCalls=1;reductionBlocks=8")
    assert ex.num_kernels == 8 and "atomicCombine<__tc::OpMin<" in ex.compiled_source
    ref = tc_oracle.run(src, "red", [X])
    assert np.array_equal(ref[0], X.min(1)) and np.array_equal(ref[1], X.max(1))
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and np.array_equal(g, r)
