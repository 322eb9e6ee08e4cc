"""The remaining workloads of the reference's benchmark suite and TC library (tc/benchmarks/*.h,
tc/library/*.h) as parity cases: name -> (tc text, entry, inputs, reduction length for the
tolerance).  An input is a shape (float32 normal values), ("int", shape, low, high) for int32
indices, or ("scalar", value) for a 0-dimensional float parameter.  Sizes are small enough for the
CPU oracle; the comprehensions are the reference's (transposed matmul tmm.cc:42-44, convolution
library/convolution.h:27, fully connected + ReLU chains library/2fcrelu.h:22, look-up tables
library/lut.h:23 and 2lut.h:23, spatial batch norm library/batchnorm.h:23, group normalisation
benchmarks/group_normalization.h:27-58, Kronecker products benchmarks/kronecker.h:124-147,
WaveNet layer benchmarks/wavenet.h:27-72)."""

TMM = """
def tmm(float(M, K) A, float(N, K) B) -> (C) {
    C(m, n) +=! A(m, r_k) * B(n, r_k)
}
"""

MATMUL = """
def matmul(float(M, K) A, float(K, N) B) -> (O) {
    O(m, n) +=! A(m, r_k) * B(r_k, n)
}
"""

# The same two products over float16 operands converted to float (no counterpart in the reference,
# whose front end has no half type): products of halves are exact in float, sums are float.
HALF_TMM = """
def half_tmm(float16(M, K) A, float16(N, K) B) -> (C) {
    C(m, n) +=! float(A(m, r_k)) * float(B(n, r_k))
}
"""
HALF_MATMUL = """
def half_matmul(float16(M, K) A, float16(K, N) B) -> (O) {
    O(m, n) +=! float(A(m, r_k)) * float(B(r_k, n))
}
"""

CONVOLUTION = """
def convolution(float(N, C, H, W) I, float(M, C, KH, KW) W1, float(M) B) -> (O) {
    O(n, m, h, w) +=! I(n, r_c, h + r_kh, w + r_kw) * W1(m, r_c, r_kh, r_kw)
    O(n, m, h, w) = O(n, m, h, w) + B(m)
}
"""

FCRELU2 = """
def func_2fcrelu(float(B, M) I, float(N, M) W1, float(N) B1, float(O, N) W2, float(O) B2) -> (O1, O2) {
    O1(b, n) +=! I(b, m) * W1(n, m)
    O1(b, n) = O1(b, n) + B1(n)
    O1(b, n) = fmax(O1(b, n), 0)
    O2(b, o) +=! O1(b, n) * W2(o, n)
    O2(b, o) = O2(b, o) + B2(o)
    O2(b, o) = fmax(O2(b, o), 0)
}
"""

# tc/benchmarks/MLP_model.cc:479-483 and :548-559
MLP1 = """
def mlp1(float(B, M) I, float(M, N) W1, float(N) B1) -> (O1) {
    O1(b, n) +=! I(b, r_m) * W1(r_m, n)
    O1(b, n) = O1(b, n) + B1(n)
    O1(b, n) = fmax(O1(b, n), 0)
}
"""

MLP3 = """
def mlp3(float(B, N) I, float(O, N) W2, float(O) B2, float(P, O) W3, float(P) B3, float(Q, P) W4, float(Q) B4)
-> (O2, O3, O4) {
    O2(b, o) +=! I(b, n) * W2(o, n)
    O2(b, o) = O2(b, o) + B2(o)
    O2(b, o) = fmax(O2(b, o), 0)
    O3(b, p) +=! O2(b, o) * W3(p, o)
    O3(b, p) = O3(b, p) + B3(p)
    O3(b, p) = fmax(O3(b, p), 0)
    O4(b, q) +=! O3(b, p) * W4(q, p)
    O4(b, q) = O4(b, q) + B4(q)
    O4(b, q) = fmax(O4(b, q), 0)
}
"""

C3 = """
def _C3(float(B, WX) I, float(WY, WX) W) -> (C3) {
    C3(b, wy) +=! I(b, r_wx) * W(wy, r_wx)
}
"""

LUT = """
def lut(float(E, D) LUT, int32(B, L) I) -> (O) {
    O(i, j) +=! LUT(I(i, k), j)
}
"""

LUT2 = """
def func_2lut(float(E1, D) LUT1, int32(B, L1) I1, float(E2, D) LUT2, int32(B, L2) I2) -> (O1, O2) {
    O1(i, j) +=! LUT1(I1(i, k), j)
    O2(i, j) +=! LUT2(I2(i, k), j)
}
"""

BATCHNORM = """
def spatialBatchNorm(float momentum, float eps, float(N, C, H, W) I, float(C) rMeanIn, float(C) rVarIn)
-> (O, rMeanOut, rVarOut, mean, centered, variance, expectedVariance, normalizedOut)
{
    mean(c) +=! I(nn, c, hh, ww)
    mean(c) = mean(c) / (N * H * W)
    rMeanOut(c) = (1 - momentum) * rMeanIn(c) + momentum * mean(c)
    centered(n, c, h, w) = I(n, c, h, w) - rMeanOut(c)
    variance(n, c, h, w) = centered(n, c, h, w) * centered(n, c, h, w)
    expectedVariance(c) +=! (variance(n, c, h, w) + eps) / (N * H * W)
    rVarOut(c) = rsqrt((1 - momentum) * rVarIn(c) + momentum * expectedVariance(c))
    O(n, c, h, w) = centered(n, c, h, w) * rVarOut(c)
    normalizedOut(n, c, h, w) = O(n, c, h, w)
}
"""

MOMENTS2 = """
def moments2_2D_1D(float(N, K) I) -> (mean, var) {
    mean(n) +=! I(n, r_k)
    var(n) +=! I(n, r_k) * I(n, r_k)
    mean(n) = mean(n) / (K)
    var(n) = var(n) / (K) - mean(n) * mean(n)
}
"""

# The single statistics of tc/benchmarks/moments.h:29-51 (the program times each of them beside the
# combined moments2_2D_1D above, moments.cc:162-303).
SUM = """
def sum_2D_1D(float(N, K) I) -> (sum) {
    sum(n) +=! I(n, r_k)
}
"""
MEAN = """
def mean_2D_1D(float(N, K) I) -> (mean) {
    mean(n) +=! I(n, r_k)
    mean(n) = mean(n) / (K)
}
"""
SUM_SQUARES = """
def sum_squares_2D_1D(float(N, K) I) -> (sum_squares) {
    sum_squares(n) +=! I(n, r_k) * I(n, r_k)
}
"""
VAR = """
def var_2D_1D(float(N, K) I, float(N) mean) -> (var) {
    var(n) +=! I(n, r_k) * I(n, r_k)
    var(n) = var(n) / (K) - mean(n) * mean(n)
}
"""
SUM_AND_SQUARES = """
def sum_and_squares_2D_1D(float(N, K) I) -> (sum, sum_squares) {
    sum(n) +=! I(n, r_k)
    sum_squares(n) +=! I(n, r_k) * I(n, r_k)
}
"""

# The three steps of the Kronecker product as comprehensions of their own (tc/benchmarks/kronecker.h:124-140).
KRONECKER3_1 = """
def Kronecker3_1(float(D2, N2) W2, float(M, N0, N1, N2) X) -> (XW2) {
    XW2(m, n0, n1, d2) +=! X(m, n0, n1, r_n2) * W2(d2, r_n2)
}
"""
KRONECKER3_2 = """
def Kronecker3_2(float(D1, N1) W1, float(M, N0, N1, D2) XW2) -> (XW2W1) {
    XW2W1(m, n0, d1, d2) +=! XW2(m, n0, r_n1, d2) * W1(d1, r_n1)
}
"""
KRONECKER3_3 = """
def Kronecker3_3(float(D0, N0) W0, float(M, N0, D1, D2) XW2W1) -> (Y) {
    Y(m, d0, d1, d2) +=! XW2W1(m, r_n0, d1, d2) * W0(d0, r_n0)
}
"""

GROUP_NORMALIZATION = """
def group_normalization(float(N, G, D, H, W) I, float(G, D) gamma, float(G, D) beta,
                        float(N, G) mean, float(N, G) var) -> (O) {
    O(n, g, d, h, w) = gamma(g, d) * (I(n, g, d, h, w) - mean(n, g)) * rsqrt(var(n, g) + 1e-5) + beta(g, d)
}
"""

GROUP_NORMALIZATION_SINGLE_KERNEL = """
def group_normalization_single_kernel(float(N, G, D, H, W) I, float(G, D) gamma, float(G, D) beta)
-> (O, sum, sumSquares) {
    sum(n, g) +=! I(n, g, r_d, r_h, r_w)
    sumSquares(n, g) +=! I(n, g, r_d, r_h, r_w) * I(n, g, r_d, r_h, r_w)
    O(n, g, d, h, w) = gamma(g, d)
        * (I(n, g, d, h, w) - sum(n, g) / (D * H * W))
        * rsqrt(sumSquares(n, g) / (D * H * W) - sum(n, g) * sum(n, g) / (D * H * W) / (D * H * W) + 1e-5)
        + beta(g, d)
}
"""

KRONECKER3 = """
def Kronecker3Full(float(D0, N0) W0, float(D1, N1) W1, float(D2, N2) W2, float(M, N0, N1, N2) X)
-> (Y, XW2, XW2W1) {
    XW2(m, n0, n1, d2) +=! X(m, n0, n1, r_n2) * W2(d2, r_n2)
    XW2W1(m, n0, d1, d2) +=! XW2(m, n0, r_n1, d2) * W1(d1, r_n1)
    Y(m, d0, d1, d2) +=! XW2W1(m, r_n0, d1, d2) * W0(d0, r_n0)
}
"""

WAVENET1 = """
def wavenet1(
    float(B, RESIDUAL_C, RECEPTIVE_FIELD) Data,
    float(DILATION_C, RESIDUAL_C, 2) FilterWeight,
    float(DILATION_C) FilterBias,
    float(DILATION_C, RESIDUAL_C, 2) GateWeight,
    float(DILATION_C) GateBias,
    float(RESIDUAL_C, DILATION_C) ResWeight,
    float(RESIDUAL_C) ResBias,
    float(SKIP_C, DILATION_C) SkipWeight,
    float(SKIP_C) SkipBias,
    float(DILATION_FACTOR) Dilation)
    -> (FilterOut, GateOut, NonLin, Res, Skip)
{
    FilterOut(b, dilation_c, rf) = FilterBias(dilation_c)
        where b in 0:B, dilation_c in 0:DILATION_C, rf in 0:RECEPTIVE_FIELD
    FilterOut(b, dilation_c, rf) += Data(b, r_residual_c, rf) * FilterWeight(dilation_c, r_residual_c, 1) +
        ((rf - DILATION_FACTOR >= 0) ?
            Data(b, r_residual_c, rf - DILATION_FACTOR) * FilterWeight(dilation_c, r_residual_c, 0) : float(0))
        where rf in 0:RECEPTIVE_FIELD
    GateOut(b, dilation_c, rf) = GateBias(dilation_c)
        where b in 0:B, dilation_c in 0:DILATION_C, rf in 0:RECEPTIVE_FIELD
    GateOut(b, dilation_c, rf) += Data(b, r_residual_c, rf) * GateWeight(dilation_c, r_residual_c, 1) +
        ((rf - DILATION_FACTOR >= 0) ?
            Data(b, r_residual_c, rf - DILATION_FACTOR) * GateWeight(dilation_c, r_residual_c, 0) : float(0))
        where rf in 0:RECEPTIVE_FIELD
    NonLin(b, dilation_c, rf) = tanh(FilterOut(b, dilation_c, rf))
        where rf in 0:RECEPTIVE_FIELD
    NonLin(b, dilation_c, rf) *= 1 / (1 + exp(-GateOut(b, dilation_c, rf)))
        where rf in 0:RECEPTIVE_FIELD
    Res(b, residual_c, rf) = Data(b, residual_c, rf) + ResBias(residual_c)
    Res(b, residual_c, rf) += NonLin(b, r_dilation_c, rf) * ResWeight(residual_c, r_dilation_c)
    Skip(b, skip, rf) +=! NonLin(b, r_dilation_c, rf) * SkipWeight(skip, r_dilation_c)
        where rf in 0:RECEPTIVE_FIELD
    Skip(b, skip, rf) = Skip(b, skip, rf) + SkipBias(skip)
        where rf in 0:RECEPTIVE_FIELD
}
"""

GROUP_CONVOLUTION = """
def group_convolution(float(N, G, C, H, W) I, float(G, F, C, KH, KW) W1, float(G, F) B) -> (O) {
    O(n, g, o, h, w) +=! I(n, g, r_i, h + r_kh, w + r_kw) * W1(g, o, r_i, r_kh, r_kw)
    O(n, g, o, h, w) = O(n, g, o, h, w) + B(g, o)
}
"""

CASES = {
    "group_convolution": (GROUP_CONVOLUTION, "group_convolution", [(2, 3, 4, 10, 9), (3, 5, 4, 3, 3), (3, 5)], 36),
    "tmm": (TMM, "tmm", [(32, 256), (128, 256)], 256),
    "half_tmm": (HALF_TMM, "half_tmm", [("half", (32, 256)), ("half", (128, 256))], 256),
    "half_matmul": (HALF_MATMUL, "half_matmul", [("half", (40, 96)), ("half", (96, 72))], 96),
    "tmm_odd": (TMM, "tmm", [(37, 70), (51, 70)], 70),
    "matmul": (MATMUL, "matmul", [(72, 60), (60, 50)], 60),
    "convolution": (CONVOLUTION, "convolution", [(3, 4, 12, 11), (8, 4, 3, 3), (8,)], 36),
    "2fcrelu": (FCRELU2, "func_2fcrelu", [(20, 48), (36, 48), (36,), (24, 36), (24,)], 48),
    "mlp1": (MLP1, "mlp1", [(20, 48), (48, 36), (36,)], 48),
    "mlp3": (MLP3, "mlp3", [(20, 24), (18, 24), (18,), (10, 18), (10,), (2, 10), (2,)], 24),
    "c3": (C3, "_C3", [(20, 48), (36, 48)], 48),
    "lut": (LUT, "lut", [(50, 24), ("int", (9, 7), 0, 50)], 7),
    "2lut": (LUT2, "func_2lut", [(50, 24), ("int", (9, 7), 0, 50), (30, 24), ("int", (9, 5), 0, 30)], 7),
    "batchnorm": (BATCHNORM, "spatialBatchNorm",
                  [("scalar", 0.1), ("scalar", 1e-5), (4, 6, 7, 5), (6,), ("positive", (6,))], 4 * 7 * 5),   # N*H*W per channel
    "moments2": (MOMENTS2, "moments2_2D_1D", [(24, 500)], 500),
    "sum": (SUM, "sum_2D_1D", [(24, 500)], 500),
    "mean": (MEAN, "mean_2D_1D", [(24, 500)], 500),
    "sum_squares": (SUM_SQUARES, "sum_squares_2D_1D", [(24, 500)], 500),
    "var": (VAR, "var_2D_1D", [(24, 500), (24,)], 500),
    "sum_and_squares": (SUM_AND_SQUARES, "sum_and_squares_2D_1D", [(24, 500)], 500),
    "kronecker3_1": (KRONECKER3_1, "Kronecker3_1", [(8, 3), (10, 5, 4, 3)], 3),
    "kronecker3_2": (KRONECKER3_2, "Kronecker3_2", [(7, 4), (10, 5, 4, 8)], 4),
    "kronecker3_3": (KRONECKER3_3, "Kronecker3_3", [(6, 5), (10, 5, 7, 8)], 5),
    "group_normalization": (GROUP_NORMALIZATION, "group_normalization",
                            [(3, 4, 5, 6, 7), (4, 5), (4, 5), (3, 4), ("positive", (3, 4))], 1),
    "group_normalization_single_kernel": (GROUP_NORMALIZATION_SINGLE_KERNEL, "group_normalization_single_kernel",
                                          [(3, 4, 5, 6, 7), (4, 5), (4, 5)], 5 * 6 * 7),   # D*H*W per (n, g)
    "kronecker3": (KRONECKER3, "Kronecker3Full", [(6, 5), (7, 4), (8, 3), (10, 5, 4, 3)], 5),
    "wavenet1": (WAVENET1, "wavenet1",
                 [(1, 8, 100), (8, 8, 2), (8,), (8, 8, 2), (8,), (8, 8), (8,), (16, 8), (16,), (2,)], 16),
    # the sizes of the program's tuned runs (wavenet.cc:139-168): eight times the skip channels,
    # dilation 1 and 32; here two batches, more skip than residual channels, dilations 1 and 5
    "wavenet1_skip256": (WAVENET1, "wavenet1",
                         [(2, 4, 50), (6, 4, 2), (6,), (6, 4, 2), (6,), (4, 6), (4,), (24, 6), (24,), (1,)], 8),
    "wavenet1_skip256_dilation32": (WAVENET1, "wavenet1",
                                    [(2, 4, 50), (6, 4, 2), (6,), (6, 4, 2), (6,), (4, 6), (4,), (24, 6), (24,), (5,)], 8),
}


# The same comprehensions at the default sizes of the reference's benchmark programs
# (tc/benchmarks/tmm.cc:42-44, MLP_model.cc:43-59 for the 1000x1024 matmul and its transposed form C3, the fc-relu chain, the one- and
# three-layer perceptrons and the one and two look-up tables, convolution.cc:40-46, group_convolution.cc:42-49, moments.cc:42-43, group_normalization.cc:42-46,
# kronecker.cc:41-47, wavenet.cc:42-60), and the mapping options the autotuner found for them on an
# MI355X (a few generations from the naive options; written relative to the naive options).
REFERENCE_SIZES = {
    "group_convolution": [(32, 32, 4, 56, 56), (32, 4, 4, 3, 3), (32, 4)],
    "tmm": [(32, 256), (128, 256)],
    "matmul": [(128, 1000), (1000, 1024)],
    "convolution": [(32, 4, 56, 56), (4, 4, 3, 3), (4,)],
    "2fcrelu": [(128, 2000), (128, 2000), (128,), (64, 128), (64,)],
    "mlp1": [(128, 2000), (2000, 128), (128,)],
    "mlp3": [(128, 128), (64, 128), (64,), (32, 64), (32,), (2, 32), (2,)],
    "c3": [(128, 1000), (1024, 1000)],
    "lut": [(100000, 64), ("int", (128, 50), 0, 100000)],
    "2lut": [(100000, 64), ("int", (128, 50), 0, 100000), (100000, 64), ("int", (128, 50), 0, 100000)],
    "moments2": [(1024, 36864)],
    "sum": [(1024, 36864)],
    "mean": [(1024, 36864)],
    "sum_squares": [(1024, 36864)],
    "var": [(1024, 36864), (1024,)],
    "sum_and_squares": [(1024, 36864)],
    "kronecker3_1": [(32, 16), (256, 16, 16, 16)],
    "kronecker3_2": [(32, 16), (256, 16, 16, 32)],
    "kronecker3_3": [(32, 16), (256, 16, 32, 32)],
    "group_normalization": [(32, 32, 16, 48, 48), (32, 16), (32, 16), (32, 32), ("positive", (32, 32))],
    "group_normalization_single_kernel": [(32, 32, 16, 48, 48), (32, 16), (32, 16)],
    "kronecker3": [(32, 16), (32, 16), (32, 16), (256, 16, 16, 16)],
    "wavenet1": [(1, 32, 4000), (32, 32, 2), (32,), (32, 32, 2), (32,), (32, 32), (32,), (32, 32), (32,), (1,)],
    "wavenet1_skip256": [(1, 32, 4000), (32, 32, 2), (32,), (32, 32, 2), (32,), (32, 32), (32,), (256, 32), (256,), (1,)],
    "wavenet1_skip256_dilation32": [(1, 32, 4000), (32, 32, 2), (32,), (32, 32, 2), (32,), (32, 32), (32,), (256, 32), (256,), (32,)],
}
TUNED_AT_REFERENCE_SIZES = {
    # one (n, g) image per block and half its rows per block in z, the 4x56x56 input window in LDS,
    # 54 threads along w; hand-set: the search's thread counts do not contain 54 x 9
    "group_convolution": "naive;tile=1,1,4,27,0;mapToThreads=54,9;mapToBlocks=32,32,8;useSharedMemory=1;unroll=16;"
                         "useReadOnlyCache=1",
    "tmm": "naive;tile=8,8;unroll=128;matchLibraryCalls=1;mapToThreads=256;mapToBlocks=256,32;useSharedMemory=1;"
           "useReadOnlyCache=1;sharedDepth=7;collapseContiguous=0;useMfma=1;"
           "outerScheduleFusionStrategy=Preserve3Coincident;intraTileScheduleFusionStrategy=Min",
    # two 16x16 tiles per block of 8 wavefronts, 250 reduction steps of a tile split over 4 of them
    "matmul": "naive;tile=16,32;unroll=256;matchLibraryCalls=1;mapToThreads=256,2;mapToBlocks=125,1000;useSharedMemory=1;"
              "useReadOnlyCache=1;vectorWidth=2;useMfma=1",
    "convolution": "naive;intraTileScheduleFusionStrategy=Min;fixParametersBeforeScheduling=1;tile=1,27,1,0;unroll=128;"
                   "tileImperfectlyNested=1;mapToThreads=256,1;mapToBlocks=256,64,1;useSharedMemory=1;useReadOnlyCache=1;"
                   "collapseContiguous=0",
    # one 16x16 tile per block, the 500 reduction steps of the first layer split over 16 wavefronts
    "2fcrelu": "naive;tile=16,16,128;unroll=256;mapToThreads=512,2;mapToBlocks=512,256;useMfma=1;useReadOnlyCache=1;"
               "useSharedMemory=1",
    "mlp1": "naive;tile=16,16,128;unroll=256;mapToThreads=64,4;mapToBlocks=512,256;useMfma=1;useReadOnlyCache=1",
    # the three layers in one kernel, 16 batch rows per block, each layer's result handed on in LDS
    "mlp3": "naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Max;tile=16,256;unroll=16;mapToThreads=256;"
            "mapToBlocks=256,128;useSharedMemory=1;unrollCopyShared=1;sharedDepth=4;useMfma=1;prefetchShared=1",
    # two 16x16 tiles per block, the 250 reduction steps of a tile split over two wavefronts each
    # reduction tiles of 200 (five of them) staged through two LDS copies: 7.6 -> 6.4 us
    "c3": "naive;tile=16,32,200;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;prefetchShared=1;"
          "useReadOnlyCache=1",
    "lut": "naive;outerScheduleFusionStrategy=Min;tile=4,32,32;unroll=64;usePrivateMemory=1;unrollCopyShared=1;"
           "collapseContiguous=0",
    "2lut": "naive;tile=2,32,32;unroll=256;mapToThreads=64,4,1;mapToBlocks=100000,256;vectorWidth=4;useMfma=1",
    "moments2": "naive;outerScheduleFusionStrategy=Max;tile=1,0;unroll=32;matchLibraryCalls=1;mapToThreads=512;mapToBlocks=1024,1;"
                "usePrivateMemory=1;useReadOnlyCache=1;vectorWidth=4",
    # 576 threads x float4 = one 48x48 plane per pass: the normalising stage then finds every
    # element in the register cache the two reductions filled (one read of the input); two groups
    # per block
    "group_normalization_single_kernel": "naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Preserve3Coincident;"
                                         "tile=1,2,0;unroll=128;matchLibraryCalls=1;mapToThreads=576;mapToBlocks=256,256;"
                                         "useSharedMemory=1;usePrivateMemory=1;useReadOnlyCache=1;vectorWidth=4",
    "group_normalization": "naive;tile=4,1,0,0,0;unroll=16;mapToThreads=48,16,1;mapToBlocks=256,256;useSharedMemory=1;"
                           "useReadOnlyCache=1;vectorWidth=4",
    "kronecker3": "naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Max;tile=1,16,0,0,8;unroll=8;"
                  "tileImperfectlyNested=1;mapToThreads=64,16;mapToBlocks=256,256,256;useSharedMemory=1;useReadOnlyCache=1;"
                  "privateDepth=5;collapseContiguous=0;useMfma=1;prefetchShared=1",
    # one statistic per pass: a wavefront (or a few) per row in lanes of four reaches 7.2-7.4 TB/s
    "sum": "naive;outerScheduleFusionStrategy=Min;tile=1,0;unroll=256;matchLibraryCalls=1;mapToThreads=64;mapToBlocks=1024,1;"
           "usePrivateMemory=1;useReadOnlyCache=1;sharedDepth=3;vectorWidth=4;prefetchShared=1",
    "mean": "naive;outerScheduleFusionStrategy=Max;tile=1,0;unroll=16;matchLibraryCalls=1;mapToThreads=128;mapToBlocks=36864,256;"
            "usePrivateMemory=1;useReadOnlyCache=1;vectorWidth=4",
    "sum_squares": "naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Min;tile=1,0;unroll=256;matchLibraryCalls=1;"
                   "mapToThreads=64;mapToBlocks=36864,1;usePrivateMemory=1;useReadOnlyCache=1;vectorWidth=4;prefetchShared=1",
    "var": "naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Max;tile=2;unroll=16;matchLibraryCalls=1;"
           "mapToThreads=256,1;mapToBlocks=1024,1;useSharedMemory=1;useReadOnlyCache=1;vectorWidth=4;prefetchShared=1",
    "sum_and_squares": "naive;outerScheduleFusionStrategy=Max;tile=1,0;unroll=8;matchLibraryCalls=1;mapToThreads=256;"
                       "mapToBlocks=36864,256;usePrivateMemory=1;useReadOnlyCache=1;vectorWidth=4",
    "kronecker3_1": "naive;tile=256,0,0,2;unroll=64;mapToThreads=128,4;mapToBlocks=256,256;usePrivateMemory=1;useReadOnlyCache=1;"
                    "useMfma=1;prefetchShared=1",
    "kronecker3_2": "naive;intraTileScheduleFusionStrategy=Max;tile=1,1,256,0,64;unroll=32;mapToThreads=128;mapToBlocks=128,256,1;"
                    "useSharedMemory=1;useReadOnlyCache=1;vectorWidth=2;collapseContiguous=0;useMfma=1;prefetchShared=1",
    "kronecker3_3": "naive;tile=1,32,0,0;unroll=1;mapToThreads=128,4;mapToBlocks=256,8;useSharedMemory=1;unrollCopyShared=1;"
                    "useReadOnlyCache=1;vectorWidth=2;useMfma=1",
    "wavenet1": "naive;intraTileScheduleFusionStrategy=Max;fixParametersBeforeScheduling=1;tile=2,2000,16,1;mapToThreads=16,64;"
                "mapToBlocks=2000,256;useSharedMemory=1;usePrivateMemory=1;privateDepth=8;sharedDepth=3;vectorWidth=4;"
                "collapseContiguous=0;prefetchShared=1",
    "wavenet1_skip256": "naive;intraTileScheduleFusionStrategy=Max;fixParametersBeforeScheduling=1;tile=2,2000,16;unroll=128;"
                        "mapToThreads=16,64;mapToBlocks=2000,256;useSharedMemory=1;usePrivateMemory=1;useReadOnlyCache=1;"
                        "privateDepth=8;sharedDepth=3;collapseContiguous=0;prefetchShared=1",
    "wavenet1_skip256_dilation32": "naive;intraTileScheduleFusionStrategy=Max;fixParametersBeforeScheduling=1;tile=2,2000,16;unroll=1;"
                                   "mapToThreads=16,64;mapToBlocks=4000,256;useSharedMemory=1;usePrivateMemory=1;useReadOnlyCache=1;"
                                   "privateDepth=8;sharedDepth=3;vectorWidth=4;collapseContiguous=0;useMfma=1;prefetchShared=1",
}


# Contractions large enough to fill the device: the transposed product at the size of the reference's
# regression fixture TMM_128_1024_1024 (test/cuda/test_tc_mapper_bugs.cc:555-656) and square matrix
# products.  name -> (key of CASES, input shapes, mapping options, reduction length)
LARGE_CONTRACTIONS = {
    "tmm_128_1024_1024": ("tmm", [(128, 1024), (1024, 1024)],
                          "naive;tile=16,32,128;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                          "prefetchShared=1", 1024),
    "matmul_1024": ("matmul", [(1024, 1024), (1024, 1024)],
                    "naive;tile=64,64,32;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                    "prefetchShared=1", 1024),
    "matmul_2048": ("matmul", [(2048, 2048), (2048, 2048)],
                    "naive;tile=128,128,16;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                    "prefetchShared=1", 2048),
    # the largest size of the transposed product's tuned runs (tc/benchmarks/tmm.cc:138-140)
    "tmm_128_16384_4096": ("tmm", [(128, 4096), (16384, 4096)],
                           "naive;tile=64,128,32;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                           "prefetchShared=1", 4096),
}

LARGE_CONTRACTIONS.update({
    # float16 operands on v_mfma_f32_16x16x16_f16 (the roofline of these two is the 2.5 PFLOP/s half peak)
    "half_tmm_4096": ("half_tmm", [("half", (4096, 4096)), ("half", (4096, 4096))],
                      "naive;tile=128,256,32;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                      "prefetchShared=1", 4096),
    "half_matmul_2048": ("half_matmul", [("half", (2048, 2048)), ("half", (2048, 2048))],
                         "naive;tile=128,128,64;mapToThreads=64,8;mapToBlocks=256,256;useMfma=1;useSharedMemory=1;"
                         "prefetchShared=1", 2048),
})

# The other sizes the reference's benchmark programs run their tuned options at
# (group_convolution.cc:104-160, moments.cc:162-303, group_normalization.cc:120-180), same layout.
OTHER_REFERENCE_SIZES = {
    "group_convolution_8_8_28": ("group_convolution", [(32, 32, 8, 28, 28), (32, 8, 8, 3, 3), (32, 8)],
                                 "naive;tile=1,1,8,26,26;mapToThreads=64,8;mapToBlocks=32,32;useSharedMemory=1;useReadOnlyCache=1;"
                                 "useMfma=1", 72),
    "group_convolution_32_32_7": ("group_convolution", [(32, 32, 32, 7, 7), (32, 32, 32, 3, 3), (32, 32)],
                                  "naive;tile=4,1,0,0,8;mapToThreads=256,4;mapToBlocks=32,256;useSharedMemory=1;useReadOnlyCache=1;"
                                  "useMfma=1", 288),
    "moments2_128_2304": ("moments2", [(128, 2304)],
                          "naive;outerScheduleFusionStrategy=Max;tile=1,4096;unroll=32;matchLibraryCalls=1;mapToThreads=256;"
                          "mapToBlocks=2304,256;usePrivateMemory=1;sharedDepth=6;vectorWidth=2", 2304),
    "group_normalization_4_512_12": ("group_normalization",
                                     [(4, 32, 16, 12, 12), (32, 16), (32, 16), (4, 32), ("positive", (4, 32))],
                                     "naive;tile=1,1,0,0,0;unroll=16;mapToThreads=12,16;mapToBlocks=256,256;useSharedMemory=1;"
                                     "useReadOnlyCache=1;collapseContiguous=0", 1),
    "group_normalization_single_kernel_4_512_12": ("group_normalization_single_kernel", [(4, 32, 16, 12, 12), (32, 16), (32, 16)],
                                                   "naive;outerScheduleFusionStrategy=Max;tile=1,1,0;unroll=64;matchLibraryCalls=1;"
                                                   "mapToThreads=128,2,1;mapToBlocks=256,256;usePrivateMemory=1;vectorWidth=4",
                                                   16 * 12 * 12),
}


def _draw(rng, spec):
    import numpy as np
    if isinstance(spec[0], str):
        kind = spec[0]
        if kind == "int":
            return rng.integers(spec[2], spec[3], size=spec[1]).astype(np.int32)
        if kind == "scalar":
            return np.array(spec[1], dtype=np.float32)
        if kind == "half":
            return rng.standard_normal(spec[1], dtype=np.float32).astype(np.float16)
        if kind == "positive":
            return (rng.random(spec[1], dtype=np.float32) + 0.5).astype(np.float32)
        raise ValueError(kind)
    return rng.standard_normal(spec, dtype=np.float32)


def make_large_inputs(name, seed=2024):
    import numpy as np
    rng = np.random.Generator(np.random.Philox(seed))
    table = LARGE_CONTRACTIONS if name in LARGE_CONTRACTIONS else OTHER_REFERENCE_SIZES
    return [_draw(rng, spec) for spec in table[name][1]]


def make_inputs(name, seed=2024, reference_sizes=False):
    import numpy as np
    rng = np.random.Generator(np.random.Philox(seed))
    return [_draw(rng, spec) for spec in (REFERENCE_SIZES if reference_sizes else {name: CASES[name][2]})[name]]
