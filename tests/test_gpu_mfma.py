"""Matrix-core (v_mfma_f32_16x16x4_f32) emission for dense contractions against the oracle:
lane layout, partial tiles in M, N and K, batch variables, epilogues, accumulation into existing
outputs.  Integer-valued inputs make the comparison bit-exact."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu

MM = "def matmul(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"
TMM = "def tmm(float(M, K) A, float(N, K) B) -> (C) { C(m, n) +=! A(m, r_k) * B(n, r_k) }"


def run(src, entry, ins_np, options, outs_init=None):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    assert "__builtin_amdgcn_mfma_f32_" in ex.compiled_source
    outs = tc.prepare_outputs(src, entry, ins)
    for i, o in enumerate(outs):
        if outs_init is not None:
            o.copy_(torch.from_numpy(outs_init[i]))
        else:
            o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs]


def ints(shape, seed):
    return np.random.Generator(np.random.Philox(seed)).integers(-4, 5, size=shape).astype(np.float32)


@pytest.mark.parametrize("m,k,n", [(16, 4, 16), (16, 16, 16), (32, 8, 48), (26, 72, 26), (5, 3, 7), (17, 33, 65), (64, 130, 20)])
@pytest.mark.parametrize("waves", [1, 4])
def test_matmul_shapes_exact(m, k, n, waves):
    print(f"mfma matmul {m}x{k}x{n} waves={waves}", flush=True)
    A, B = ints((m, k), m * 100 + k), ints((k, n), n)
    opts = f"naive;tile=32,32;mapToThreads=64,{waves};mapToBlocks=64,64;useMfma=1"
    (C,) = run(MM, "matmul", [A, B], opts)
    assert np.array_equal(C, A @ B)
    (Ct,) = run(TMM, "tmm", [A, np.ascontiguousarray(B.T)], opts)
    assert np.array_equal(Ct, A @ B)


# (m, k, n, tile of n, wavefronts, operands through LDS, quarter-tile passes expected)
QUARTER_CASES = [
    (16, 8, 20, 32, 1, 0, True), (40, 36, 17, 32, 1, 0, True), (16, 16, 4, 32, 1, 0, True), (16, 16, 4, 32, 4, 1, True),
    (48, 10, 196, 0, 1, 0, True), (48, 10, 196, 0, 4, 1, True),
    # not where the busiest wavefront would get more to do, or where the reduction is divided among wavefronts
    (16, 8, 20, 32, 4, 1, False), (33, 144, 26, 32, 1, 0, False), (33, 144, 26, 32, 4, 1, False), (20, 7, 52, 28, 4, 1, False),
    (16, 64, 9, 0, 4, 1, False),
]


@pytest.mark.parametrize("m,k,n,tile_n,waves,lds,quarter", QUARTER_CASES)
def test_surplus_columns_go_through_quarter_tile_passes(m, k, n, tile_n, waves, lds, quarter):
    """Up to twelve surplus columns of a block tile are multiplied by v_mfma_f32_4x4x1 passes of
    four columns each (another lane layout for operand, result and epilogue than the 16x16 tiles):
    bit-exact on integer-valued data, row-wise epilogue operand included."""
    print(f"quarter tiles {m}x{k}x{n} tile_n={tile_n} waves={waves} lds={lds}", flush=True)
    src = """
def mmb(float(M, K) A, float(K, N) B, float(M) bias) -> (C) {
    C(m, n) +=! A(m, r_k) * B(r_k, n)
    C(m, n) = C(m, n) + bias(m)
}
"""
    A, B, bias = ints((m, k), m + k), ints((k, n), n + 7), ints((m,), 11)
    opts = f"naive;tile=16,{tile_n};mapToThreads=64,{waves};mapToBlocks=64,64;useMfma=1;useSharedMemory={lds}"
    ins = [torch.from_numpy(a).cuda() for a in (A, B, bias)]
    ex = tc.compile(src, "mmb", ins, opts)
    assert ("__builtin_amdgcn_mfma_f32_4x4x1f32" in ex.compiled_source) == quarter
    outs = tc.prepare_outputs(src, "mmb", ins)
    outs[0].fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    assert np.array_equal(outs[0].cpu().numpy(), A @ B + bias[:, None])


def test_matmul_with_lds_operands_and_untiled_problem():
    A, B = ints((50, 40), 1), ints((40, 30), 2)
    (C,) = run(MM, "matmul", [A, B], "naive;tile=0,0;mapToThreads=64,2;mapToBlocks=1;useMfma=1;useSharedMemory=1")
    assert np.array_equal(C, A @ B)


def test_accumulate_into_existing_output():
    src = "def mmacc(float(M, K) A, float(K, N) B) -> (C) { C(m, n) += A(m, r_k) * B(r_k, n) }"
    A, B = ints((20, 12), 3), ints((12, 18), 4)
    C0 = ints((20, 18), 5)
    (C,) = run(src, "mmacc", [A, B], "naive;tile=32,32;mapToThreads=64;useMfma=1", outs_init=[C0])
    assert np.array_equal(C, C0 + A @ B)


@pytest.mark.parametrize("opts", [
    "naive;tile=1,26,26;mapToThreads=64,4;mapToBlocks=500;useMfma=1",
    "naive;tile=1,26,26;mapToThreads=64,4;mapToBlocks=500;useMfma=1;useSharedMemory=1",
    "naive;tile=2,26,26;mapToThreads=64,8;mapToBlocks=500;useMfma=1;useSharedMemory=1",
])
def test_batch_matmul(opts):
    X, Y = ints((9, 26, 72), 6), ints((9, 72, 26), 7)
    (Z,) = run(W.BATCH_MATMUL, "batch_matmul", [X, Y], opts)
    assert np.array_equal(Z, np.einsum("bnm,bmk->bnk", X, Y))


@pytest.mark.parametrize("opts", [
    "naive;tile=1,1,16,14,14;mapToThreads=64,4;mapToBlocks=32,32;useMfma=1;useSharedMemory=1",
    "naive;tile=1,1,16,14,14;mapToThreads=64,2;mapToBlocks=32,32;useMfma=1",
    "naive;tile=1,2,8,7,14;mapToThreads=64,4;mapToBlocks=32,32;useMfma=1;useSharedMemory=1",
])
def test_group_convolution_with_bias_epilogue(opts):
    I, Wt, B = ints((3, 4, 6, 16, 16), 8), ints((4, 16, 6, 3, 3), 9), ints((4, 16), 10)
    (O,) = run(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B], opts)
    (ref,) = tc_oracle.run(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B])
    assert np.array_equal(O, ref)


def test_full_size_configs_within_tolerance():
    for name, opts in (("c3_batch_matmul", "naive;tile=1,26,26;mapToThreads=64,4;mapToBlocks=500;useMfma=1;useSharedMemory=1"),
                       ("c4_group_convolution", "naive;tile=1,1,16,14,14;mapToThreads=64,4;mapToBlocks=32,32;useMfma=1;useSharedMemory=1")):
        src, entry, _, _, k = W.CONFIGS[name]
        ins = W.make_inputs(name)
        got = run(src, entry, ins, opts)
        ref = tc_oracle.run(src, entry, ins)
        for g, r in zip(got, ref):
            assert np.abs(g - r).max() <= W.tolerance(k, r), name


def test_non_contractions_fall_back_to_the_vector_path():
    src = "def add(float(N, M) A, float(N, M) B) -> (C) { C(n, m) = A(n, m) + B(n, m) }"
    A = torch.randn(32, 32, device="cuda")
    ex = tc.compile(src, "add", [A, A], "naive;useMfma=1")
    assert "mfma" not in ex.compiled_source


@pytest.mark.parametrize("opts", [
    "naive;tile=1,1,16,14,14;mapToThreads=64,4;mapToBlocks=3,2;useMfma=1;useSharedMemory=1;prefetchShared=1",
    "naive;tile=1,1,16,14,14;mapToThreads=64,4;mapToBlocks=2,4;useMfma=1;useSharedMemory=1;prefetchShared=1",
    "naive;tile=1,1,16,14,14;mapToThreads=64,2;mapToBlocks=1,1;useMfma=1;useSharedMemory=1;prefetchShared=1",
])
def test_prefetched_lds_staging_matches(opts):
    """Software-pipelined staging: blocks loop over several tiles, loading the next tile's
    footprints while the current one is computed."""
    I, Wt, B = ints((3, 4, 6, 16, 16), 18), ints((4, 16, 6, 3, 3), 19), ints((4, 16), 20)
    ins = [torch.from_numpy(a).cuda() for a in (I, Wt, B)]
    ex = tc.compile(W.GROUP_CONVOLUTION, "group_convolution", ins, opts)
    assert "more_" in ex.compiled_source
    (O,) = tc.prepare_outputs(W.GROUP_CONVOLUTION, "group_convolution", ins)
    O.fill_(float("nan"))
    tc.run(ex, ins, [O])
    torch.cuda.synchronize()
    (ref,) = tc_oracle.run(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B])
    assert np.array_equal(O.cpu().numpy(), ref)


def test_prefetched_lds_staging_on_the_vector_path():
    X, Y = ints((9, 26, 72), 26), ints((9, 72, 26), 27)
    opts = "naive;tile=1,26,26,72;mapToThreads=26,13;mapToBlocks=2;unroll=4;useSharedMemory=1;prefetchShared=1"
    ins = [torch.from_numpy(a).cuda() for a in (X, Y)]
    ex = tc.compile(W.BATCH_MATMUL, "batch_matmul", ins, opts)
    assert "more_" in ex.compiled_source and "mfma" not in ex.compiled_source
    (Z,) = tc.prepare_outputs(W.BATCH_MATMUL, "batch_matmul", ins)
    tc.run(ex, ins, [Z])
    torch.cuda.synchronize()
    assert np.array_equal(Z.cpu().numpy(), np.einsum("bnm,bmk->bnk", X, Y))


@pytest.mark.parametrize("opts", [
    "naive;tile=64,64,32;mapToThreads=64,4;mapToBlocks=256,256;useMfma=1;useSharedMemory=1",
    "naive;tile=32,48,16;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1",
    "naive;tile=64,32,24;mapToThreads=64,2;mapToBlocks=256,256;useMfma=1;useSharedMemory=0",
    "naive;tile=16,16,7;mapToThreads=64,4;mapToBlocks=256,256;useMfma=1;useSharedMemory=1",   # 7 does not divide 192: untiled
    # software pipeline over the reduction tiles: the next tile's operands load while this one multiplies
    "naive;tile=64,64,32;mapToThreads=64,4;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1",
    "naive;tile=32,48,16;mapToThreads=64,8;mapToBlocks=3,2;useMfma=1;useSharedMemory=1;prefetchShared=1",
])
def test_reduction_tiling_stages_operands_per_tile(opts):
    """The outermost reduction index may be tiled: operands are staged in LDS once per reduction
    tile and the accumulators of a wavefront's output tiles stay in registers across the loop."""
    src = "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"
    rng = np.random.Generator(np.random.Philox(41))
    A = rng.integers(-3, 4, size=(200, 192)).astype(np.float32)
    B = rng.integers(-3, 4, size=(192, 150)).astype(np.float32)
    ins = [torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()]
    ex = tc.compile(src, "mm", ins, opts)
    (C,) = tc.prepare_outputs(src, "mm", ins)
    C.fill_(float("nan"))
    tc.run(ex, ins, [C])
    torch.cuda.synchronize()
    assert np.array_equal(C.cpu().numpy(), A @ B)                 # small integers: exact in fp32
    tiled = "for (int t_r_k" in ex.compiled_source
    assert tiled == (",7;" not in opts)
    assert ("pk_A_" in ex.compiled_source or "pk0_A_" in ex.compiled_source) == ("prefetchShared=1" in opts)
    # accumulate into an existing output across reduction tiles
    acc = "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) += A(m, r_k) * B(r_k, n) }"
    ex = tc.compile(acc, "mm", ins, opts)
    C0 = rng.integers(-5, 6, size=(200, 150)).astype(np.float32)
    C = torch.from_numpy(C0.copy()).cuda()
    tc.run(ex, ins, [C])
    torch.cuda.synchronize()
    assert np.array_equal(C.cpu().numpy(), C0 + A @ B)


FC = """def fc(float(B, K) I, float(N, K) W1, float(N) B1) -> (O1) {
    O1(b, n) +=! I(b, k) * W1(n, k)
    O1(b, n) = O1(b, n) + B1(n)
    O1(b, n) = fmax(O1(b, n), 0) }"""


ROTATED_CASES = [
    # (M, N, K, tile, wavefronts, register stages the tile loop is unrolled by)
    (128, 128, 64, "64,64,32", 8, 1),     # two reduction tiles
    (128, 128, 96, "64,64,32", 8, 1),     # three: an odd number of tiles keeps one stage
    (128, 128, 128, "64,64,32", 4, 2),
    (128, 128, 256, "64,64,32", 8, 4),
    (100, 72, 160, "32,32,32", 4, 1),     # partial row and column tiles, five reduction tiles
    (200, 136, 1000, "64,32,40", 4, 1),   # 25 reduction tiles of 10 steps
    (64, 192, 384, "64,64,16", 8, 4),     # 24 tiles of 4 steps
    (256, 256, 512, "128,128,16", 8, 4),
]


@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("m,n,k,tile,waves,stages", ROTATED_CASES)
def test_rotated_pipeline_with_register_stages_is_exact(m, n, k, tile, waves, stages, transposed):
    """Register-blocked, reduction-tiled products with two LDS copies: the operand values of the
    next tile's first half are read behind the barrier while this tile's second half multiplies,
    and the loads of up to four tiles are in flight (past the last tile they fetch it again)."""
    src = ("def mm(float(M, K) A, float(N, K) B) -> (C) { C(m, n) +=! A(m, r_k) * B(n, r_k) }" if transposed else
           "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }")
    rng = np.random.Generator(np.random.Philox(43))
    A = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
    B = rng.integers(-3, 4, size=((n, k) if transposed else (k, n))).astype(np.float32)
    ins = [torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()]
    opts = f"naive;tile={tile};mapToThreads=64,{waves};mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1"
    print(f"case {m}x{n}x{k} tile {tile} waves {waves} transposed {transposed}", flush=True)
    ex = tc.compile(src, "mm", ins, opts)
    source = ex.compiled_source
    assert "pk0_A_" in source and "ra_[" in source, "not the rotated, register-blocked form"
    assert (f"pk{stages - 1}_A_" in source) and (f"pk{stages}_A_" not in source), "number of register stages"
    (C,) = tc.prepare_outputs(src, "mm", ins)
    C.fill_(float("nan"))
    tc.run(ex, ins, [C])
    torch.cuda.synchronize()
    assert np.array_equal(C.cpu().numpy(), A @ (B.T if transposed else B))     # small integers: exact in fp32


@pytest.mark.parametrize("k,opts,split", [
    # one tile, 16 wavefronts, 128 steps: 16 slices of 8
    (512, "naive;tile=16,16;mapToThreads=512,2;mapToBlocks=64,64;useMfma=1", 16),
    # 250 steps over 8 wavefronts per tile: 7 slices of 32 and one of 26
    (1000, "naive;tile=16,32;mapToThreads=512,2;mapToBlocks=64,64;useMfma=1", 8),
    # operands staged in LDS per reduction tile, the slices inside every tile
    (1000, "naive;tile=16,32,200;mapToThreads=512,2;mapToBlocks=64,64;useMfma=1;useSharedMemory=1", 6),
    (1000, "naive;tile=16,16,200;mapToThreads=256,1;mapToBlocks=64,64;useMfma=1;useSharedMemory=1;prefetchShared=1", 4),
    # blocks loop over tiles: the partial tiles in LDS are reused from one iteration to the next
    (512, "naive;tile=16,16;mapToThreads=256,2;mapToBlocks=2,3;useMfma=1", 8),
    # a reduction whose length is no multiple of 4 lanes groups x steps
    (203, "naive;tile=16,16;mapToThreads=256;mapToBlocks=64,64;useMfma=1", 4),
])
def test_reduction_split_over_wavefronts(k, opts, split):
    """Fewer output tiles than wavefronts: the reduction steps of a tile are divided among several
    wavefronts whose partial tiles meet in LDS."""
    A, B = ints((40, k), k), ints((k, 70), k + 1)
    ins = [torch.from_numpy(a).cuda() for a in (A, B)]
    src = tc.compile(MM, "matmul", ins, opts).compiled_source
    assert "ksplit0_" in src and f"sl_ < {split})" in src, src
    (C,) = run(MM, "matmul", [A, B], opts)
    assert np.array_equal(C, A @ B)


def test_split_reduction_accumulates_into_existing_output_and_runs_the_epilogue():
    src = "def mmacc(float(M, K) A, float(K, N) B) -> (C) { C(m, n) += A(m, r_k) * B(r_k, n) }"
    A, B, C0 = ints((20, 400), 3), ints((400, 18), 4), ints((20, 18), 5)
    opts = "naive;tile=16,16;mapToThreads=256,2;mapToBlocks=8,8;useMfma=1"
    (C,) = run(src, "mmacc", [A, B], opts, outs_init=[C0])
    assert np.array_equal(C, C0 + A @ B)
    I, W1, B1 = ints((30, 600), 6), ints((50, 600), 7), ints((50,), 8)
    (O,) = run(FC, "fc", [I, W1, B1], opts)
    assert np.array_equal(O, np.maximum(I @ W1.T + B1, 0))
    (ref,) = tc_oracle.run(FC, "fc", [I, W1, B1])
    assert np.array_equal(O, ref)


HALF_MM = "def hmm(float16(M, K) A, float16(K, N) B) -> (C) { C(m, n) +=! float(A(m, r_k)) * float(B(r_k, n)) }"
HALF_TMM = "def htmm(float16(M, K) A, float16(N, K) B) -> (C) { C(m, n) +=! float(A(m, r_k)) * float(B(n, r_k)) }"
HALF_BMM = """def hbmm(float16(B, N, M) X, float16(B, M, K) Y, float(K) bias) -> (Z) {
    Z(b, n, k) +=! float(X(b, n, r_m)) * float(Y(b, r_m, k))
    Z(b, n, k) = Z(b, n, k) + bias(k) }"""

HALF_CASES = [
    # (text, entry, shapes of the half operands, options, half-precision matrix instruction expected)
    # rotated pipeline, eight steps a tile: two v_mfma_f32_16x16x16_f16 per tile and pair of output tiles
    (HALF_MM, "hmm", [(256, 256), (256, 256)],
     "naive;tile=64,64,32;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1", True),
    (HALF_TMM, "htmm", [(128, 512), (256, 512)],
     "naive;tile=64,128,32;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1", True),
    # reduction tiles of 64 and of 16 steps of four: the halves of a tile hold whole groups, or they do not
    (HALF_MM, "hmm", [(128, 384), (384, 128)],
     "naive;tile=64,64,64;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1", True),
    (HALF_MM, "hmm", [(128, 192), (192, 160)],
     "naive;tile=32,32,16;mapToThreads=64,4;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1", False),
    # partial tiles on every side, operands through LDS without reduction tiles, and straight from memory
    (HALF_MM, "hmm", [(100, 90), (90, 70)],
     "naive;tile=32,32;mapToThreads=64,4;mapToBlocks=256,256;useMfma=1;useSharedMemory=1", False),
    (HALF_MM, "hmm", [(100, 90), (90, 70)], "naive;tile=16,32;mapToThreads=64,2;mapToBlocks=256,256;useMfma=1", False),
    (HALF_TMM, "htmm", [(37, 1000), (45, 1000)],
     "naive;tile=16,32;unroll=256;mapToThreads=256,2;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;vectorWidth=2", False),
    # a batch index and an epilogue in float
    (HALF_BMM, "hbmm", [(7, 26, 72), (7, 72, 26)],
     "naive;tile=1,26,26;mapToThreads=64,4;mapToBlocks=500;useMfma=1;useSharedMemory=1", False),
]


@pytest.mark.parametrize("src,entry,shapes,options,half_instruction", HALF_CASES)
def test_float16_operands_on_the_matrix_cores(src, entry, shapes, options, half_instruction):
    """`float(A) * float(B)` of float16 tensors is a contraction the matrix cores take: operands
    are staged and read as halves, products and sums are float.  Small integers make every sum
    exact, so the result equals numpy's in every bit; normal deviates stay within the tolerance of
    a float sum against the oracle (which multiplies the converted values in float)."""
    rng = np.random.Generator(np.random.Philox(71))
    ins = [rng.integers(-4, 5, size=s).astype(np.float16) for s in shapes]
    extra = [rng.integers(-3, 4, size=(shapes[1][-1],)).astype(np.float32)] if entry == "hbmm" else []
    ex_source = {}

    def go(arrays):
        ins_t = [torch.from_numpy(a).cuda() for a in arrays]
        ex = tc.compile(src, entry, ins_t, options)
        ex_source["text"] = ex.compiled_source
        outs = tc.prepare_outputs(src, entry, ins_t)
        outs[0].fill_(float("nan"))
        tc.run(ex, ins_t, outs)
        torch.cuda.synchronize()
        return outs[0].cpu().numpy()

    got = go(ins + extra)
    text = ex_source["text"]
    assert ("__builtin_amdgcn_mfma_f32_16x16x16f16" in text) == half_instruction
    assert half_instruction or "__builtin_amdgcn_mfma_f32_16x16x4f32" in text
    a, b = ins[0].astype(np.float64), ins[1].astype(np.float64)
    if entry == "hmm":
        exact = a @ b
    elif entry == "htmm":
        exact = a @ b.T
    else:
        exact = np.einsum("bnm,bmk->bnk", a, b) + extra[0]
    assert got.dtype == np.float32 and np.array_equal(got, exact.astype(np.float32))
    (ref,) = tc_oracle.run(src, entry, ins + extra)
    assert np.array_equal(ref, got)
    normal = [rng.standard_normal(s).astype(np.float16) for s in shapes]
    got = go(normal + extra)
    (ref,) = tc_oracle.run(src, entry, normal + extra)
    k = shapes[0][-1]
    assert np.abs(got - ref).max() <= 1e-5 * np.sqrt(k) * max(float(np.abs(ref).max()), 1.0)
