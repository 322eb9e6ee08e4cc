"""Mapper known answers on a GPU-less host: tightened launch bounds, stage/kernel formation under
the fusion strategies, reduction-library matching, LDS promotion footprints, collapsing, vector
lanes, error paths.  Scenarios follow test/test_cuda_mapper.cc (:352-383 Basic, :632-645 1-D code on
a 2-D mapping, :837-850/:930-994 reductions) and test_cuda_mapper_memory_promotion.cc (:298-310
footprints, :441-449), restated for this mapper's output."""
import re

import pytest

import tensorcomprehensions_amd as tc
from tensorcomprehensions_amd import MappingOptions, ShapeOnly
from tests import workloads as W


def mapped(src, entry, shapes, options):
    return tc.map_only(src, entry, [ShapeOnly(s) for s in shapes], options)


ADD = "def fun(float(N, M) A, float(N, M) B) -> (C) { C(n, m) = A(n, m) + B(n, m) }"


def test_launch_bounds_are_tightened_to_the_problem():
    o = MappingOptions.naive().tile(16, 16).mapToBlocks(256, 256).mapToThreads(16, 16).collapseContiguous(False)
    src, launches = mapped(ADD, "fun", [(512, 40), (512, 40)], o)
    assert launches == [((32, 3, 1), (16, 16, 1))]            # 512/16 blocks in x, ceil(40/16) in y
    # the last m tile is partial: a guard must protect it
    assert "<= 39" in src


def test_one_dimensional_code_on_a_two_dimensional_mapping():
    src, launches = mapped("def f(float(N) A) -> (B) { B(n) = A(n) }", "f", [(100,)], MappingOptions.naive())
    (grid, block), = launches
    assert grid == (4, 1, 1) and block == (32, 1, 1)          # tile 32 -> 4 tiles; y extents collapse to 1


def test_kernel_name_and_argument_order():
    src, _ = mapped(W.TENSORDOT, "tensordot", [(16, 8, 16, 17, 25), (16, 16, 2, 17, 25)], "naive")
    # sizes appended in parameter-name order C1,C2,C3,H,N,W; args: sizes, outputs, inputs
    assert re.search(r"tensordot_8_16_2_17_16_25\(int C1, int C2, int C3, int H, int N, int W, "
                     r"float\* __restrict__ pO, const float\* __restrict__ pI0, const float\* __restrict__ pI1\)", src)


def test_collapse_and_vector_lanes():
    shapes = [(4, 8, 8, 28, 28), (4, 8, 2, 28, 28)]
    src, _ = mapped(W.TENSORDOT, "tensordot", shapes, MappingOptions.naive().vectorWidth(4))
    assert "i_h_w_o" in src and "i_h_w_v" in src              # h,w merged (784 contiguous), split in lanes of 4
    src, _ = mapped(W.TENSORDOT, "tensordot", shapes, MappingOptions.naive().collapseContiguous(False))
    assert "i_h_w" not in src and "i_w" in src
    # 17*25 = 425 is not a multiple of 4: lanes are dropped, the code stays scalar
    src, _ = mapped(W.TENSORDOT, "tensordot", [(2, 3, 4, 17, 25), (2, 4, 2, 17, 25)], MappingOptions.naive().vectorWidth(4))
    assert "i_h_w" in src and "i_h_w_v" not in src
    # the convolution's h and w are not jointly contiguous in the input (windows): no merge
    src, _ = mapped(W.GROUP_CONVOLUTION, "group_convolution", [(2, 2, 4, 8, 8), (2, 4, 4, 3, 3), (2, 4)], "naive")
    assert "i_h_w" not in src


def test_reduction_library_is_matched_only_when_asked():
    red = "def fun(float(N, K) I) -> (O) { O(n) +=! I(n, r_k) }"
    src, launches = mapped(red, "fun", [(64, 4096)], MappingOptions.naive().matchLibraryCalls(True).mapToThreads(128, 2).tile(2))
    assert "__tc::blockAllReduceX<__tc::OpSum<float>, 128, 2, 1>" in src
    assert launches == [((32, 1, 1), (128, 2, 1))]
    src, _ = mapped(red, "fun", [(64, 4096)], MappingOptions.naive().matchLibraryCalls(False).mapToThreads(128, 2))
    assert "blockAllReduceX" not in src
    # x extent 1: nothing to reduce across
    src, _ = mapped(red, "fun", [(64, 4096)], MappingOptions.naive().matchLibraryCalls(True).mapToThreads(1))
    assert "blockAllReduceX" not in src
    # min / max / product use their own operators
    mx = "def fun(float(N, K) I) -> (O) { O(n) max=! I(n, r_k) }"
    src, _ = mapped(mx, "fun", [(64, 4096)], MappingOptions.naive().matchLibraryCalls(True).mapToThreads(64))
    assert "__tc::OpMax<float>" in src


def test_lds_promotion_footprints():
    o = MappingOptions.naive().tile(1, 26, 26, 72).mapToThreads(26, 13).mapToBlocks(500).unroll(4).useSharedMemory(True)
    src, launches = mapped(W.BATCH_MATMUL, "batch_matmul", [(500, 26, 72), (500, 72, 26)], o)
    assert launches == [((500, 1, 1), (26, 13, 1))]
    # per block: X[1][26][72] and Y[1][72][26] (footprint = min(tile, size) per dimension)
    assert "float lds0_X[1872];" in src
    assert re.search(r"float lds0_Y\[(1872|1944)\];", src)
    # a barrier after the copies; none before them: nothing has read LDS ahead of the first copy of
    # a kernel whose blocks do not loop over tiles
    assert src.count("__syncthreads();") == 1
    looped, _ = mapped(W.BATCH_MATMUL, "batch_matmul", [(500, 26, 72), (500, 72, 26)], o.mapToBlocks(100))
    assert looped.count("__syncthreads();") == 2              # the next tile's copy waits for this tile's readers
    # without the switch nothing is staged
    src, _ = mapped(W.BATCH_MATMUL, "batch_matmul", [(500, 26, 72), (500, 72, 26)], o.useSharedMemory(False))
    assert "__shared__" not in src
    # no reuse, no promotion: a point-wise sum reads every element once
    src, _ = mapped(ADD, "fun", [(64, 64), (64, 64)], MappingOptions.naive().useSharedMemory(True))
    assert "__shared__" not in src


def test_convolution_window_footprint_includes_the_halo():
    o = "naive;tile=1,1,16,14,14,4;mapToThreads=14,14;mapToBlocks=32,32;unroll=16;useSharedMemory=1"
    src, _ = mapped(W.GROUP_CONVOLUTION, "group_convolution", [(32, 32, 16, 16, 16), (32, 16, 16, 3, 3), (32, 16)], o)
    # input tile: 4 channels x (14+2) x (14+2)
    assert "float lds0_I[1024];" in src
    # the weights are read at the same address by every thread of the block (f is not mapped to
    # threads here): they go through the scalar cache, not LDS
    assert "lds0_W1" not in src


def test_lds_budget_is_respected():
    o = MappingOptions.naive().tile(1, 26, 26, 72).mapToThreads(26, 13).mapToBlocks(500).unroll(4).useSharedMemory(True)
    src, _ = mapped(W.BATCH_MATMUL, "batch_matmul", [(500, 26, 72), (500, 72, 26)], o.maxSharedMemory(8000))
    assert src.count("__shared__ ") == 1                      # only one of the two 7.5 KB tiles fits


def test_fusion_strategies_decide_kernel_count():
    gc = [(2, 3, 4, 9, 8), (3, 5, 4, 3, 3), (3, 5)]
    _, launches = mapped(W.GROUP_CONVOLUTION, "group_convolution", gc, MappingOptions.naive())
    assert len(launches) == 1                                  # bias epilogue fused into the reduction stage
    _, launches = mapped(W.GROUP_CONVOLUTION, "group_convolution", gc, MappingOptions.naive().scheduleFusionStrategy("Min"))
    assert len(launches) == 2
    src, launches = mapped(W.MOMENTS, "moments", [(64, 1024)], MappingOptions.naive())
    # every thread owns whole rows: var re-reads the mean its own thread stored, no barrier
    assert len(launches) == 1 and "// stage 1: var" in src
    assert "__syncthreads" not in src and "wave_barrier" not in src
    # reduction spread over threadIdx.x: lane 0 stores the mean the other threads read
    rowwise = MappingOptions.naive().tile(1).mapToBlocks(64).matchLibraryCalls(True)
    src, launches = mapped(W.MOMENTS, "moments", [(64, 1024)], rowwise.mapToThreads(64))
    assert launches == [((64, 1, 1), (64, 1, 1))]                  # one wavefront: ordering only, no s_barrier
    between = src[src.index("// stage 0: mean"):src.index("// stage 1: var")]
    assert between.count("__builtin_amdgcn_wave_barrier();") == 1 and "__syncthreads" not in between
    src, launches = mapped(W.MOMENTS, "moments", [(64, 1024)], rowwise.mapToThreads(256))
    assert launches == [((64, 1, 1), (256, 1, 1))]
    between = src[src.index("// stage 0: mean"):src.index("// stage 1: var")]
    tail = between[between.rindex("pmean["):]                       # after the store of the mean
    assert tail.count("__syncthreads();") == 1 and "wave_barrier" not in between
    _, launches = mapped(W.MOMENTS, "moments", [(64, 1024)], MappingOptions.naive().scheduleFusionStrategy("Min"))
    assert len(launches) == 2


def test_barriers_between_stages_only_where_threads_exchange_data():
    """Role of insertBestSyncInSeq (mapped_scop.cc:729-770) on the stage sequence of a kernel."""
    chain = """def f(float(N, M) A) -> (O, P) {
        O(i, j) = A(i, j) + 1.0
        P(i, j) = O(i, j) * 2.0 }"""
    src, launches = mapped(chain, "f", [(64, 64)], MappingOptions.naive())
    assert len(launches) == 1 and "// stage 1: P" in src
    assert "__syncthreads" not in src and "wave_barrier" not in src      # same thread produces and consumes
    mirrored = """def g(float(N, M) A) -> (O, P) {
        O(i, j) = A(i, j) + 1.0
        P(i, j) = O(i, j) * 2.0 + O(i, M - 1 - j) }"""
    src, launches = mapped(mirrored, "g", [(64, 64)], MappingOptions.naive().tile(32, 64).mapToThreads(64, 4))
    if len(launches) == 1:                                             # fused: the mirrored read crosses threads
        assert src.count("__syncthreads();") == 1


def test_producer_consumer_matmuls_share_only_the_row_dimension():
    two = """def fun(float(M, K) I, float(K, N) W1, float(N, P) W2) -> (O1, O2) {
        O1(m, n) +=!  I(m, r_k) * W1(r_k, n)
        O2(m, p) +=! O1(m, r_n) * W2(r_n, p) }"""
    shapes = [(64, 32), (32, 48), (48, 16)]
    src, launches = mapped(two, "fun", shapes, MappingOptions.naive().scheduleFusionStrategy("Max").tile(4, 16).mapToBlocks(256, 256))
    assert len(launches) == 1
    (grid, _), = launches
    assert grid == (16, 1, 1)                                  # blocks only over m: O2 needs whole rows of O1
    _, launches = mapped(two, "fun", shapes, MappingOptions.naive())   # Preserve3Coincident: needs 2 shared dims
    assert len(launches) == 2


@pytest.mark.parametrize("bad,fragment", [
    ("naive;mapToThreads=0", "mapping to 0"),
    ("naive;mapToBlocks=0", "mapping to 0"),
    ("naive;mapToThreads=1024,2;tile=0,0;collapseContiguous=0", "exceeds the device limit"),
])
def test_options_the_mapper_cannot_honour(bad, fragment):
    with pytest.raises(tc.TcError) as e:
        mapped(ADD, "fun", [(2048, 2048), (2048, 2048)], bad)
    assert fragment in str(e.value)


def test_generated_sources_compile_for_gfx950():
    cases = [
        (W.MOMENTS, "moments", [(64, 1000)], "naive;matchLibraryCalls=1;mapToThreads=96,2;tile=2"),
        (W.BATCH_MATMUL, "batch_matmul", [(7, 26, 72), (7, 72, 26)], "naive;tile=1,13,26,8;mapToThreads=26,13;useSharedMemory=1;unroll=8"),
        ("def f(int32(N) A, float(N) B) -> (C) { C(n) = float(A(n) % 3) * B(n) + exp(B(n)) }", "f", [(100,), (100,)], "pointwise"),
    ]
    for src, entry, shapes, opts in cases:
        ins = [ShapeOnly(s, "int32" if (src.startswith("def f(int32") and i == 0) else "float32") for i, s in enumerate(shapes)]
        ex = tc.compile(src, entry, ins, opts)
        assert ex.num_kernels >= 1 and "extern \"C\" __global__" in ex.compiled_source


def test_block_axis_order_keeps_sharing_blocks_on_one_xcd():
    """Blocks that share an operand must not differ in blockIdx.x (consecutive ids go to different
    XCDs): the group convolution's weights depend on g only, so g takes x and n the slower axis; the
    tensordot's small operand depends on n, which already is the x axis."""
    src, launches = mapped(W.GROUP_CONVOLUTION, "group_convolution", W.CONFIGS["c4_group_convolution"][2],
                           W.TUNED["c4_group_convolution"])
    assert "const int t_g = blockIdx.x;" in src and "const int t_n = blockIdx.y;" in src
    assert launches[0][0] == (32, 32, 1)
    src, launches = mapped(W.TENSORDOT, "tensordot", W.CONFIGS["c2_tensordot"][2], W.TUNED["c2_tensordot"])
    assert "const int t_n = blockIdx.x;" in src and launches[0][0] == (32, 64, 1)
    # x extent not a multiple of 8: left alone
    src, _ = mapped(W.GROUP_CONVOLUTION, "group_convolution", [(6, 5, 4, 9, 8), (5, 6, 4, 3, 3), (5, 6)],
                    "naive;tile=1,1,8,7,6;mapToThreads=64,2;mapToBlocks=6,5")
    assert "const int t_n = blockIdx.x;" in src


def wavenet_source(options):
    from tests import benchmark_tcs as B
    src, entry, shapes, _ = B.CASES["wavenet1"]
    return mapped(src, entry, shapes, options)


def test_register_cache_holds_only_what_every_stage_loop_shares():
    """The cache of an operand read by several stages holds one tile: with tile loops that each
    stage runs by itself (maximal fusion, no block mapping of rf) nothing is cached; with the loops
    opened around all stages the unconditional read of Data is, and the read that the
    comprehension guards with `rf - DILATION_FACTOR >= 0` never moves ahead of its guard."""
    common = "naive;tile=1,16,4;mapToThreads=2,3,3;mapToBlocks=64,3;unroll=8;useSharedMemory=0;usePrivateMemory=1"
    src, _ = wavenet_source(common + ";outerScheduleFusionStrategy=Max")
    assert "for (int t_rf = 0; t_rf < 25; ++t_rf)" in src and "rcache" not in src
    src, _ = wavenet_source(common)
    assert "rcache0_[a_ * 8 + (0) * 8 + q_r_residual_c] = pData[800 * i_b + 100 * i_r_residual_c + i_rf];" in src
    assert "rcache1_" not in src
    assert "? (pData[800 * i_b + 100 * i_r_residual_c + i_rf - 2] *" in src


def test_kernel_with_a_matrix_core_stage_runs_whole_wavefronts():
    """A matrix-core stage reads threadIdx.x as the lane and threadIdx.y as the wavefront: the
    other stages of its kernel are mapped onto that 64 x waves block instead of widening it."""
    src, launches = wavenet_source("naive;tile=2;mapToThreads=128;mapToBlocks=16;matchLibraryCalls=1;useMfma=1;"
                                   "useSharedMemory=0;outerScheduleFusionStrategy=Max")
    assert launches == [((1, 1, 1), (64, 2, 1))]
    assert "v_mfma_f32_16x16x4_f32" in src and "blockAllReduceX<__tc::OpSum<float>, 64, 2, 1>" in src


def test_pointwise_stage_reads_the_reductions_register_cache():
    """Normalise-after-moments in one kernel: the reductions run over one merged variable
    (r_d, r_h, r_w collapse), the normalising stage over (d, h*w); with 576 threads x 4 lanes every
    thread meets the same element at the same slot in all three stages, so the input is read
    once.  With 512 threads the forms differ and the last stage reads memory again."""
    from tests import benchmark_tcs as B
    src, entry, _, _ = B.CASES["group_normalization_single_kernel"]
    shapes = B.REFERENCE_SIZES["group_normalization_single_kernel"]
    common = ("naive;tile=1,1;mapToBlocks=32,32;matchLibraryCalls=1;vectorWidth=4;unroll=64;usePrivateMemory=1;"
              "outerScheduleFusionStrategy=Max;mapToThreads=")
    text, launches = mapped(src, entry, shapes, common + "576")
    assert launches == [((32, 32, 1), (576, 1, 1))]
    assert text.count("pI[") == 1 and "float rcache0_[64];" in text
    assert "(rcache0_[a_] - (rfwd0_sum / " in text           # the sums come in registers as well
    text, _ = mapped(src, entry, shapes, common + "512")
    assert text.count("pI[") == 2


def test_a_later_rewrite_of_a_tensor_joins_the_kernel_of_its_producer():
    """One-pass moments: mean and var are reduced, then rescaled by two pointwise statements that
    do not follow their reductions directly.  Every subscript of both tensors is the shared row
    variable, so all four stages form one kernel."""
    from tests import benchmark_tcs as B
    text, launches = mapped(B.MOMENTS2, "moments2_2D_1D", [(64, 512)],
                            "naive;tile=1;mapToThreads=128;mapToBlocks=64;matchLibraryCalls=1;outerScheduleFusionStrategy=Max")
    assert launches == [((64, 1, 1), (128, 1, 1))]
    assert [ln.strip() for ln in text.split("\n") if ln.strip().startswith("// stage")] == [
        "// stage 0: mean", "// stage 1: var", "// stage 2: mean", "// stage 3: var"]
    # a rewrite over a variable the stages do not share stays in the kernel too, behind a barrier:
    # other threads wrote the elements it reads
    rows = """def f(float(N, M) A) -> (S, T) {
        S(n, m) = A(n, m)
        T(n) +=! A(n, m)
        S(n, m) = S(n, m) / T(n)
    }"""
    text, launches = mapped(rows, "f", [(64, 512)], "naive;tile=1;mapToThreads=128;mapToBlocks=64;outerScheduleFusionStrategy=Max")
    assert len(launches) == 1
    body = text[text.index("// stage 1: T"):text.index("// stage 2: S")]
    assert "__syncthreads();" in body


def test_tuned_options_of_the_five_workloads_compile_with_the_expected_launches():
    """The options bench.py uses (tests/workloads.py:TUNED) map to the launch shapes the
    measurements quote, and hipRTC compiles them for gfx950 without a GPU."""
    expected = {
        "c1_tensordot_small": [((16, 8, 1), (425, 1, 1))],
        "c2_tensordot": [((32, 64, 1), (196, 1, 1))],
        "c3_batch_matmul": [((500, 1, 1), (64, 4, 1))],
        "c4_group_convolution": [((32, 32, 1), (64, 4, 1))],
        "c5_moments": [((1024, 1, 1), (512, 1, 1))],
    }
    for name, launches in expected.items():
        src, entry, shapes = W.CONFIGS[name][0], W.CONFIGS[name][1], W.CONFIGS[name][2]
        ex = tc.compile(src, entry, [ShapeOnly(s) for s in shapes], W.TUNED[name])
        assert [ex.launch_bounds(k) for k in range(ex.num_kernels)] == launches, name


TWO_CONVOLUTIONS = """
def two(float(N,C,H,W) I, float(O,C,KH,KW) W1, float(O,C,KH,KW) W2) -> (A, B) {
    A(n, o, h, w) +=! I(n, c, h + kh, w + kw) * W1(o, c, kh, kw)
    B(n, o, h, w) +=! I(n, c, h + kh, w + kw) * W2(o, c, kh, kw)
}
"""
STENCIL = ("def blur(float(N, M) A) -> (O) { O(i, j) = (A(i, j) + A(i, j + 1) + A(i, j + 2) + "
           "A(i + 1, j) + A(i + 1, j + 1) + A(i + 1, j + 2)) / 6.0 }")


def test_stages_of_a_kernel_share_one_staged_copy_of_a_footprint():
    """Two stages that read the same window of the same input (the reference forms one reference
    group per tensor and scope, tc/core/polyhedral/memory_promotion.cc:63-321): one LDS array, one
    copy, the second stage only addresses it."""
    options = "naive;tile=1,8,10,10;mapToThreads=10,10;mapToBlocks=4;unroll=8;useSharedMemory=1;outerScheduleFusionStrategy=Max"
    src, launches = mapped(TWO_CONVOLUTIONS, "two", [(4, 3, 12, 12), (8, 3, 3, 3), (8, 3, 3, 3)], options)
    assert len(launches) == 1
    assert src.count("__shared__") == 1 and "lds0_I[432]" in src and "lds1_I" not in src
    assert len(re.findall(r"lds0_I\[[^\]]*\] = stage_", src)) == 1          # copied once
    stage1 = src[src.index("// stage 1: B"):]
    assert "lds0_I[" in stage1 and "pI[" not in stage1                         # read from the shared copy
    # kept apart, each kernel stages its own
    src2, launches2 = mapped(TWO_CONVOLUTIONS, "two", [(4, 3, 12, 12), (8, 3, 3, 3), (8, 3, 3, 3)],
                             options.replace("outerScheduleFusionStrategy=Max", "outerScheduleFusionStrategy=Min"))
    assert len(launches2) == 2 and src2.count("__shared__") == 2


def test_a_stage_without_a_reduction_stages_overlapping_windows():
    """Promotion is decided by reuse, not by the kind of statement: six accesses per element of a
    (tile + halo) window (memory_promotion_heuristic.cc:211-244, 'has reuse')."""
    options = "naive;tile=8,64;mapToThreads=64,2;mapToBlocks=16,16;unroll=4;useSharedMemory=1"
    src, _ = mapped(STENCIL, "blur", [(100, 200)], options)
    assert "__shared__ __attribute__((aligned(16))) float lds0_A[594];" in src           # (8 + 1) x (64 + 2)
    body = src[src.index("acc_[a_] = ("):]
    assert body.count("lds0_A[") >= 6 and "pA[" not in body.split("\n")[0]
    # no reuse, no staging
    src2, _ = mapped(ADD, "fun", [(100, 200), (100, 200)], options)
    assert "__shared__" not in src2


def test_offsets_are_64_bit_once_a_tensor_reaches_2_to_the_31_elements():
    """Element offsets are formed in 64 bits when some tensor has 2^31 elements or more; every
    single extent still has to stay below 2^31 (loop variables are int)."""
    big = "def big(int8(M, N) X) -> (s, Y) { s(m) +=! int32(X(m, n))\n Y(m, n) = int8(X(m, n) + 1) }"
    opts = "naive;tile=4,1024;mapToThreads=256;mapToBlocks=256,32;unroll=4"
    src, _ = tc.map_only(big, "big", [ShapeOnly((65544, 32768), "int8")], opts)
    assert "(int64)32768 * " in src
    small, _ = tc.map_only(big, "big", [ShapeOnly((655, 32768), "int8")], opts)
    assert "(int64)" not in small
    with pytest.raises(tc.TcError) as e:
        tc.map_only("def f(int8(N) A) -> (B) { B(i) = A(i) }", "f", [ShapeOnly((2 ** 31 + 8,), "int8")], "naive")
    assert "dimension of 2^31 or more" in str(e.value)


def test_outputs_with_a_lower_bound_are_stored_from_it():
    """Element k of a shifted dimension holds the point min + k: the write and every later read of
    the tensor subtract the bound (inferred by test/test_inference.cc:158-186)."""
    src, _ = mapped("def fun(float(I_0) I) -> (O, P) { O(i) = I(i - 1)\n P(j) = O(j + 1) }", "fun", [(100,)], "naive")
    assert "pO[i_i] = " in src and "acc_[a_] = pI[i_i];" in src     # i shifted to 0..99, I(i - 1) with it
    assert "acc_[a_] = pO[i_i];" in src and "pP[i_i] = " in src     # P(j) reads point j + 1 = element j


def test_promotion_for_coalescing_alone():
    """An operand without reuse is staged when the threads along x walk a slower dimension of it
    (memory_promotion_heuristic.cc:211-244), and not when they walk its rows."""
    o = "naive;tile=32,32;mapToThreads=32,8;mapToBlocks=128,128;unroll=4;useSharedMemory=1"
    src, _ = mapped("def tr(float(N, M) A) -> (O) { O(j, i) = A(i, j) }", "tr", [(4096, 4096)], o)
    assert "lds0_A[1056]" in src                        # 32 x 32 tile, pitch 33
    src, _ = mapped("def cp(float(N, M) A) -> (O) { O(i, j) = A(i, j) }", "cp", [(4096, 4096)], o)
    assert "lds0_A" not in src


def test_every_scalar_type_maps_including_half():
    """The type sweep of test/test_tc2halide.cc:201-222, with the float16 it leaves out (the
    reference's front end refuses the type, tc/lang/sema.h:62-66; hipRTC needs no header for it)."""
    spelled = {"bool": "bool", "uint8": "unsigned char", "uint16": "unsigned short", "uint32": "unsigned int",
               "uint64": "unsigned long long", "int8": "signed char", "int16": "short", "int32": "int", "int64": "long long",
               "float16": "_Float16", "float32": "float", "float64": "double", "float": "float", "double": "double"}
    for name, c in spelled.items():
        dtype = {"float": "float32", "double": "float64"}.get(name, name)
        src, _ = tc.map_only(f"def test_type({name}(N) A) -> (B) {{ B(k) +=! A(i) where k in 0:1 }}", "test_type",
                             [ShapeOnly((100,), dtype)], "naive")
        assert f"const {c}* __restrict__ pA" in src, name


def test_written_tensor_is_forwarded_to_later_stages_through_lds():
    """Producer -> consumer through LDS (the reference promotes written references and copies them
    out, memory_promotion.cc:507-524): the producer stores to memory and to the block's copy, the
    reader indexes the copy; a barrier closes each iteration of a kernel-level loop."""
    chain = """def chain(float(M, K) A, float(K, N) W) -> (B, C) {
        B(m, k) = A(m, k) * 2.0 + 1.0
        C(m, n) +=! B(m, r_k) * W(r_k, n) }"""
    base = "naive;tile=4,32;mapToThreads=32,4;outerScheduleFusionStrategy=Max;unroll=4"
    src, launches = mapped(chain, "chain", [(40, 48), (48, 70)], base + ";mapToBlocks=64;useSharedMemory=1")
    assert len(launches) == 1 and "float fwd0_B[192];" in src                    # 4 rows x 48
    assert "pB[i_k + 48 * i_m] = acc_[a_]; fwd0_B[((i_m) - (0 + 4 * t_m)) * 48 + ((i_k) - (0))] = acc_[a_];" in src
    assert "(fwd0_B[((i_m) - (0 + 4 * t_m)) * 48 + ((i_r_k_s1) - (0))] * " in src and "pB[" not in src.split("// stage 1")[1]
    looped, _ = mapped(chain, "chain", [(40, 48), (48, 70)], base + ";mapToBlocks=3;useSharedMemory=1")
    assert looped.count("__syncthreads();") == src.count("__syncthreads();") + 1
    plain, _ = mapped(chain, "chain", [(40, 48), (48, 70)], base + ";mapToBlocks=64;useSharedMemory=0")
    assert "fwd0_B" not in plain


def test_block_wide_reduction_result_is_forwarded_in_a_register():
    """usePrivateMemory: what a block-wide reduction leaves in every thread is read by the later
    stages of the kernel from a register (the reference promotes written scalars to registers,
    memory_promotion_heuristic.cc:581-616); thread 0 still stores it, and no barrier stands between
    the stages for its sake."""
    moments = """def moments(float(M, N) X) -> (mean, var) {
        mean(m) +=! X(m, r_n) / N
        var(m) +=! (X(m, r_n) - mean(m)) * (X(m, r_n) - mean(m)) / N }"""
    base = "naive;tile=1;mapToThreads=128;matchLibraryCalls=1;outerScheduleFusionStrategy=Max"
    src, launches = mapped(moments, "moments", [(37, 1000)], base + ";mapToBlocks=64;usePrivateMemory=1")
    assert launches == [((37, 1, 1), (128, 1, 1))]
    stage1 = src.split("// stage 1")[1]
    assert "float rfwd0_mean;" in src and "rfwd0_mean = acc_[a_]; if (ok_ && threadIdx.x == 0)" in src
    assert "- rfwd0_mean)" in stage1 and "pmean[" not in stage1
    plain, _ = mapped(moments, "moments", [(37, 1000)], base + ";mapToBlocks=64;usePrivateMemory=0")
    assert "rfwd0_mean" not in plain and "pmean[" in plain.split("// stage 1")[1]
    assert plain.count("__syncthreads();") == src.count("__syncthreads();") + 1
    # blocks that loop over rows: the register is set anew in every iteration
    looped, launches = mapped(moments, "moments", [(37, 1000)], base + ";mapToBlocks=8;usePrivateMemory=1")
    assert launches[0][0] == (8, 1, 1) and "rfwd0_mean" in looped
    # rows along threadIdx.y, one per thread: every thread keeps the result of its own row, and a
    # block whose rows are single wavefronts needs no block barrier at all
    rows, launches = mapped(moments, "moments", [(37, 1000)],
                            base.replace("tile=1", "tile=4").replace("mapToThreads=128", "mapToThreads=64,4") + ";mapToBlocks=64;usePrivateMemory=1")
    assert launches == [((10, 1, 1), (64, 4, 1))] and "- rfwd0_mean)" in rows.split("// stage 1")[1]
    kernel = rows[rows.index('extern "C"'):]
    assert "__syncthreads();" not in kernel and "const int p_m = (int)threadIdx.y;" in kernel
    # two rows per thread: the register would have to be an array indexed like the reader's loop
    two = base.replace("tile=1", "tile=2") + ";mapToBlocks=64;usePrivateMemory=1"
    assert "rfwd0_mean" not in mapped(moments, "moments", [(37, 1000)], two)[0]
    # a second row of threads that only the reader uses would reduce nothing but identities
    spread = """def spread(float(M, N) X) -> (s, Y) {
        s(m) +=! X(m, r_n)
        Y(m, j, n) = X(m, n) - s(m) where j in 0:4 }"""
    src, launches = mapped(spread, "spread", [(37, 256)],
                           "naive;tile=1,4,0;mapToThreads=64,4;mapToBlocks=64;matchLibraryCalls=1;usePrivateMemory=1;outerScheduleFusionStrategy=Max")
    assert launches[0][1][1] == 4 and "rfwd0_s" not in src


def test_in_place_updates_of_a_forwarded_reduction_stay_in_the_register():
    """`mean(n) = mean(n) / K` after the sum (tc/benchmarks/moments.h:52-59) works on the register
    every thread holds; the last writer alone stores, and no barrier or reload separates the four
    statements."""
    moments2 = """def moments2(float(N, K) I) -> (mean, var) {
        mean(n) +=! I(n, r_k)
        var(n) +=! I(n, r_k) * I(n, r_k)
        mean(n) = mean(n) / (K)
        var(n) = var(n) / (K) - mean(n) * mean(n) }"""
    opts = "naive;tile=1,0;mapToThreads=128;mapToBlocks=64;matchLibraryCalls=1;outerScheduleFusionStrategy=Max"
    src, launches = mapped(moments2, "moments2", [(37, 1000)], opts + ";usePrivateMemory=1")
    assert launches == [((37, 1, 1), (128, 1, 1))]
    kernel = src[src.index('extern "C"'):]
    assert "__syncthreads();" not in kernel
    stage0, stage1, stage2, stage3 = kernel.split("// stage ")[1:]
    assert "rfwd0_mean = acc_[a_];" in stage0 and "pmean[" not in stage0
    assert "rfwd1_var = acc_[a_];" in stage1 and "pvar[" not in stage1
    assert "acc_[a_] = rfwd0_mean;" in stage2 and "rfwd0_mean = acc_[a_]; if (ok_) pmean[i_n] = acc_[a_];" in stage2
    assert "acc_[a_] = rfwd1_var;" in stage3 and "(rfwd0_mean * rfwd0_mean)" in stage3
    assert "if (ok_) pvar[i_n] = acc_[a_];" in stage3 and "pmean[" not in stage3
    plain, _ = mapped(moments2, "moments2", [(37, 1000)], opts + ";usePrivateMemory=0")
    assert "rfwd" not in plain and "acc_[a_] = pmean[" in plain and "__syncthreads();" in plain[plain.index('extern "C"'):]
    # an update that is itself a reduction, or that runs over more points than the block holds,
    # is not an update of the held element
    again = """def again(float(N, K) I) -> (s) {
        s(n) +=! I(n, r_k)
        s(n) += I(n, r_k) * I(n, r_k) }"""
    assert "rfwd" not in mapped(again, "again", [(37, 1000)], opts + ";usePrivateMemory=1")[0]


def test_reduction_blocks_divides_a_sum_among_blocks():
    """reductionBlocks: `O +=! f` becomes a zeroing kernel and a kernel whose outermost parallel
    variable numbers slices of the outermost reduction index; partial sums meet in atomics."""
    src = "def bias_grad(float(N, M, H, W) d_O) -> (d_B) { d_B(m) +=! d_O(r_n, m, r_h, r_w) }"
    opts = "naive;tile=1,1;mapToThreads=256;mapToBlocks=64,64;matchLibraryCalls=1"
    plain, launches = mapped(src, "bias_grad", [(32, 64, 56, 56)], opts)
    assert launches == [((64, 1, 1), (256, 1, 1))] and "atomicAccumulate(&p" not in plain
    split, launches = mapped(src, "bias_grad", [(32, 64, 56, 56)], opts + ";reductionBlocks=16")
    assert launches == [((1, 1, 1), (16, 1, 1)), ((16, 64, 1), (256, 1, 1))]  # a fill of 64 floats, then 16 slices x 64 outputs
    assert "__tc::atomicAccumulate(&pd_B[i_m], acc_[a_]);" in split
    assert "401408 * i_slice0" in split                                       # slice = 2 of the 32 images
    # an extent without a divisor in range, a narrow element type, a maximum: mapped as without the option
    for text, shape, dtype, blocks in [("def f(float(M, K) X) -> (s) { s(m) +=! X(m, r_k) }", (8, 127), "float32", 64),
                                       ("def f(int8(M, K) X) -> (s) { s(m) +=! X(m, r_k) }", (8, 128), "int8", 16),
                                       ("def f(float(M, K) X) -> (s) { s(m) max=! X(m, r_k) }", (8, 128), "float32", 16)]:
        s, _ = tc.map_only(text, "f", [ShapeOnly(shape, dtype)], f"naive;reductionBlocks={blocks}")
        assert "atomicAccumulate(&p" not in s
    # the option survives text and wire form
    o = MappingOptions("naive;reductionBlocks=8")
    assert "reductionBlocks=8" in o.normalized() and "reductionBlocks" not in MappingOptions("naive").normalized()


def test_strided_accesses_are_staged_without_the_elements_jumped_over():
    """test/test_cuda_mapper_memory_promotion.cc:709-751: O(i, j) = I(j, 2 * i + 1) promotes a
    32 x 32 footprint with stride 2 along the second dimension (stride 5 for I(j, 5 * i)); the copy
    reads the tensor with that stride, the computation reads the staged array without it."""
    opts = "naive;tile=32,32;mapToThreads=32,8;mapToBlocks=64,64;useSharedMemory=1;unroll=4"
    for sub, step in (("2 * i + 1", 2), ("5 * i", 5)):
        src, _ = mapped("def strided(float(N, M) I) -> (O) { O(i, j) = I(j, %s) }" % sub, "strided", [(42, 420)], opts)
        assert "float lds0_I[1056];" in src                                   # 32 rows of 32 (+1: odd pitch)
        assert f"const int g1_ = lo0_I_1 + l1_ * {step};" in src              # strided read of the tensor
        assert f" - lo0_I_1) / {step}];" in src                                # unit stride in the staged array


def test_double_math_results_are_pinned_before_a_conditional_combine():
    """hipcc (ROCm 7.0 and 7.2) does not finish compiling `r = tanh(x); if (c) acc = max(acc, r)` in
    double precision inside the reduction loops of a partial tile; the generated code pins the
    value in a register first (an empty asm), and the definition JIT-compiles in a second."""
    import time
    text = """def f(double(P, K) A) -> (O0, O1) {
        O0(j, i) = A(i, j)
        O1(i) max=! tanh(O0(i, j)) }"""
    src, _ = tc.map_only(text, "f", [ShapeOnly((70, 33), "float64")], "naive")
    assert 'double r_ = tanh(' in src and 'asm volatile("" : "+v"(r_));' in src
    single, _ = mapped(text.replace("double", "float"), "f", [(70, 33)], "naive")
    assert 'asm volatile("" : "+v"(r_));' not in single.split('extern "C"', 1)[1]
    # the JIT step in a child process under a time limit: a recurrence of the defect fails this
    # test instead of hanging the suite (hipRTC needs no device)
    import os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (f"import sys; sys.path.insert(0, {root!r}); import tensorcomprehensions_amd as tc; "
            f"tc.compile({text!r}, 'f', [tc.ShapeOnly((70, 33), 'float64')], 'naive'); print('compiled')")
    t0 = time.time()
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "compiled" in r.stdout, r.stderr[-2000:]
    assert time.time() - t0 < 60
