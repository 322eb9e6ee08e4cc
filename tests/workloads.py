"""The five benchmark TCs, their shapes, seeded inputs and the tolerance rule shared by tests,
the smoke check and the benchmark."""
import math

import numpy as np

TENSORDOT = """
def tensordot(float(N, C1, C2, H, W) I0, float(N, C2, C3, H, W) I1) -> (O) {
    O(n, c1, c3, h, w) +=! I0(n, c1, r_c2, h, w) * I1(n, r_c2, c3, h, w)
}
"""
BATCH_MATMUL = """
def batch_matmul(float(B, N, M) X, float(B, M, K) Y) -> (Z) {
    Z(b, n, k) +=! X(b, n, mm) * Y(b, mm, k)
}
"""
GROUP_CONVOLUTION = """
def group_convolution(float(N,G,C,H,W) I, float(G,F,C,KH,KW) W1, float(G,F) B) -> (O) {
    O(n, g, f, h, w) +=! I(n, g, c, h + kh, w + kw) * W1(g, f, c, kh, kw)
    O(n, g, f, h, w) = O(n, g, f, h, w) + B(g, f)
}
"""
MOMENTS = """
def moments(float(M, N) X) -> (mean, var) {
    mean(m) +=! X(m, r_n) / N
    var(m) +=! (X(m, r_n) - mean(m)) * (X(m, r_n) - mean(m)) / N
}
"""

# name -> (tc, entry, input shapes, distribution, reduction length)
CONFIGS = {
    "c1_tensordot_small": (TENSORDOT, "tensordot", [(16, 8, 16, 17, 25), (16, 16, 2, 17, 25)], "uniform", 16),
    "c2_tensordot": (TENSORDOT, "tensordot", [(32, 512, 8, 28, 28), (32, 8, 2, 28, 28)], "normal", 8),
    "c3_batch_matmul": (BATCH_MATMUL, "batch_matmul", [(500, 26, 72), (500, 72, 26)], "normal", 72),
    "c4_group_convolution": (GROUP_CONVOLUTION, "group_convolution",
                             [(32, 32, 16, 16, 16), (32, 16, 16, 3, 3), (32, 16)], "normal", 144),
    "c5_moments": (MOMENTS, "moments", [(1024, 32768)], "normal", 32768),
}

# Hand-picked mapping options per config (starting points of the tuner, also used by the benchmark).
TUNED = {
    "c1_tensordot_small": "naive;tile=1,1,0,0,0;mapToThreads=425;mapToBlocks=256,256;unroll=128;vectorWidth=4;useReadOnlyCache=1",
    "c2_tensordot": "naive;tile=1,8,2,0;mapToThreads=256;mapToBlocks=32,64;unroll=128;vectorWidth=4;useReadOnlyCache=1",
    "c3_batch_matmul": "naive;tile=1,26,26;mapToThreads=64,4;mapToBlocks=500;useMfma=1;useSharedMemory=1",
    "c4_group_convolution": "naive;tile=1,1,16,14,14;mapToThreads=64,4;mapToBlocks=32,32;useMfma=1;useSharedMemory=1;useReadOnlyCache=1",
    "c5_moments": "naive;tile=1;mapToThreads=512;mapToBlocks=1024;matchLibraryCalls=1;unroll=8;vectorWidth=4;usePrivateMemory=1;useReadOnlyCache=1",
}


def make_inputs(name, seed=0xC0FFEE):
    """Seeded inputs from a counter-based generator (Philox), identical on every machine."""
    _, _, shapes, dist, _ = CONFIGS[name]
    rng = np.random.Generator(np.random.Philox(seed))
    out = []
    for s in shapes:
        if dist == "uniform":
            out.append(rng.random(s, dtype=np.float32))
        else:
            out.append(rng.standard_normal(s, dtype=np.float32))
    return out


def tolerance(reduction_length, ref):
    """fp32 bound of the acceptance rule: 1e-5 * sqrt(K) * max|ref|."""
    return 1e-5 * math.sqrt(reduction_length) * max(float(np.abs(ref).max()), 1e-30)
