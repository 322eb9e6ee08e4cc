"""Outputs whose inferred lower bound is not zero (test/test_inference.cc:158-186 shifts, :213-240
convolution gradient, :243-266 padded convolution; the reference's tests only infer them).
Storage starts at the bound: element k of a dimension holds the point min + k.  The oracle is
pinned on closed forms first, then the HIP path is held to it."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu

PADDED = """def convolution(float(N,C,H,W) I, float(M,C,KH,KW) W1) -> (pad, tmp) {
    pad(n, c, h, w)  = I(n, c, h - 2 - 3, w - 3 - 4)
    tmp(n, m, h, w) +=! pad(n, c, 2 * h + kh, 3 * w + kw) * W1(m, c, kh, kw) }"""
GRAD = """def convolutionGrad(float(N,C,H,W) I, float(M,C,KH,KW) W1, float(N,M,OH,OW) d_O) -> (d_I, d_W1, d_B) {
    d_I(n, c, h, w) +=! d_O(n, m, h - kh, w - kw) * W1(m, c, kh, kw)
    d_W1(m, c, kh, kw) +=! d_O(n, m, h - kh, w - kw) * I(n, c, h, w)
    d_B(m) +=! d_O(n, m, h, w) }"""
WHERE = """def f(float(N, M) A) -> (O, P) {
    O(i, j) = A(i, j) * 2.0 where i in 3:N, j in 1:5
    P(i) +=! O(i, j) + A(i - 3, j) }"""

OPTIONS = [
    "naive",
    "naive;tile=2,2,4,4;mapToThreads=8,4;mapToBlocks=4,4;unroll=4;useSharedMemory=1;outerScheduleFusionStrategy=Max",
    "naive;tile=1,4,0,0;mapToThreads=16,4;mapToBlocks=8;unroll=2;vectorWidth=2;matchLibraryCalls=1",
    "naive;tile=4,8;mapToThreads=64;mapToBlocks=256;collapseContiguous=1;useReadOnlyCache=1",
]


def run(src, entry, ins_np, options):
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs]


@pytest.mark.parametrize("options", OPTIONS)
@pytest.mark.parametrize("stmt", ["O(i) = I(i - 1)", "O(i) = I(i + 5)", "O(i) = I(i - 1) + float(i)"])
def test_shift_1d(stmt, options):
    src = "def fun(float(I_0) I) -> (O) { %s }" % stmt
    I = np.random.Generator(np.random.Philox(5)).standard_normal(1000, dtype=np.float32)
    (ref,) = tc_oracle.run(src, "fun", [I])
    # point p of O lives in element p - min: every element is the input element beside it
    assert np.array_equal(ref, I + np.arange(1, 1001, dtype=np.float32) if "float(i)" in stmt else I)
    (got,) = run(src, "fun", [I], options)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("options", OPTIONS)
def test_padded_convolution(options):
    N, C, H, Wd, M, KH, KW = 2, 3, 20, 31, 4, 3, 5
    rng = np.random.Generator(np.random.Philox(6))
    I = rng.integers(-3, 4, size=(N, C, H, Wd)).astype(np.float32)
    W1 = rng.integers(-3, 4, size=(M, C, KH, KW)).astype(np.float32)
    pad, tmp = tc_oracle.run(PADDED, "convolution", [I, W1])
    assert np.array_equal(pad, I) and tmp.shape == (N, M, (H - KH + 1) // 2, (Wd - KW + 1) // 3)
    closed = np.zeros(tmp.shape, np.float32)
    for h in range(tmp.shape[2]):
        for w in range(tmp.shape[3]):
            hp, wp = h + 3, w + 3                      # tmp's own bounds start at (3, 3)
            patch = I[:, :, 2 * hp - 5:2 * hp - 5 + KH, 3 * wp - 7:3 * wp - 7 + KW]
            closed[:, :, h, w] = np.einsum("nckl,mckl->nm", patch, W1)
    assert np.array_equal(tmp, closed)                  # small integers: exact in any order
    got = run(PADDED, "convolution", [I, W1], options)
    assert np.array_equal(got[0], pad) and np.array_equal(got[1], tmp)


@pytest.mark.parametrize("options", OPTIONS)
def test_convolution_gradient_with_a_larger_output_gradient(options):
    N, C, H, Wd, M, KH, KW, OH, OW = 2, 3, 12, 13, 4, 3, 5, 14, 14
    rng = np.random.Generator(np.random.Philox(7))
    ins = [rng.integers(-3, 4, size=s).astype(np.float32)
           for s in [(N, C, H, Wd), (M, C, KH, KW), (N, M, OH, OW)]]
    an = tc_oracle.analyze(GRAD, "convolutionGrad", [a.shape for a in ins])
    assert [list(an.tensors[o].mins) for o in an.outputs] == [[0, 0, KH - 1, KW - 1], [0, 0, H - OH, Wd - OW], [0]]
    ref = tc_oracle.run(GRAD, "convolutionGrad", ins)
    got = run(GRAD, "convolutionGrad", ins, options)
    for g, r in zip(got, ref):
        assert g.shape == r.shape and np.array_equal(g, r)


@pytest.mark.parametrize("options", OPTIONS)
def test_where_clause_lower_bounds(options):
    A = np.random.Generator(np.random.Philox(8)).integers(-9, 10, size=(40, 7)).astype(np.float32)
    O, P = tc_oracle.run(WHERE, "f", [A])
    assert np.array_equal(O, 2 * A[3:, 1:5])
    assert np.array_equal(P, (2 * A[3:, 1:5] + A[:37, 1:5]).sum(1))
    got = run(WHERE, "f", [A], options)
    assert np.array_equal(got[0], O) and np.array_equal(got[1], P)
