"""Pins the CPU oracle: golden loop nests of the reference (test/test_core.cc:93-232), the library
routines the reference's own tests use as ground truth (bmm, conv2d(groups), einsum, mean/var:
tc/benchmarks/batchmatmul.cc:67, group_convolution.cc:87-101, moments.cc:54-59,
test/test_mapper_llvm.cc:182-262), float64 brute force, exact integer sums and closed forms."""
import re

import numpy as np
import pytest
import torch

from oracle import tc_oracle
from tests import workloads as W


def nest(src, entry, shapes, sym=None):
    an = tc_oracle.analyze(src, entry, shapes)
    return tc_oracle.emit_loop_nest_text(an, sym)


def test_loop_nest_two_matmul_golden():
    src = """
def fun(float(M, K) I, float(K, N) W1, float(N, P) W2) -> (O1, O2) {
    O1(m, n) +=!  I(m, r_k) * W1(r_k, n)
    O2(m, p) +=! O1(m, r_n) * W2(r_n, p)
}
"""
    sym = {("O1", "m"): "M", ("O1", "n"): "N", ("O1", "r_k"): "K", ("O2", "m"): "M", ("O2", "p"): "P", ("O2", "r_n"): "N"}
    expected = """for (int O1_s0_m = 0; O1_s0_m < M; O1_s0_m++) {
  for (int O1_s0_n = 0; O1_s0_n < N; O1_s0_n++) {
    O1[O1_s0_m][O1_s0_n] = 0.000000f;
  }
}
for (int O1_s1_m = 0; O1_s1_m < M; O1_s1_m++) {
  for (int O1_s1_n = 0; O1_s1_n < N; O1_s1_n++) {
    for (int O1_s1_r_k = 0; O1_s1_r_k < K; O1_s1_r_k++) {
      O1[O1_s1_m][O1_s1_n] = (O1[O1_s1_m][O1_s1_n] + (I[O1_s1_m][O1_s1_r_k]*W1[O1_s1_r_k][O1_s1_n]));
    }
  }
}
for (int O2_s0_m = 0; O2_s0_m < M; O2_s0_m++) {
  for (int O2_s0_p = 0; O2_s0_p < P; O2_s0_p++) {
    O2[O2_s0_m][O2_s0_p] = 0.000000f;
  }
}
for (int O2_s1_m = 0; O2_s1_m < M; O2_s1_m++) {
  for (int O2_s1_p = 0; O2_s1_p < P; O2_s1_p++) {
    for (int O2_s1_r_n = 0; O2_s1_r_n < N; O2_s1_r_n++) {
      O2[O2_s1_m][O2_s1_p] = (O2[O2_s1_m][O2_s1_p] + (O1[O2_s1_m][O2_s1_r_n]*W2[O2_s1_r_n][O2_s1_p]));
    }
  }
}
"""
    assert nest(src, "fun", [(3, 4), (4, 5), (5, 6)], sym) == expected


def test_loop_nest_group_convolution_golden():
    src = """
def fun(float(N, G, C, H, W) I1, float(G, C, F, KH, KW) W1) -> (O1) {
    O1(n, g, f, h, w) +=! I1(n, g, r_c, h + r_kh, w + r_kw) * W1(g, r_c, f, r_kh, r_kw)
}
"""
    sym = {("O1", "n"): "N", ("O1", "g"): "G", ("O1", "f"): "F", ("O1", "h"): "((H - KH) + 1)",
           ("O1", "w"): "((W - KW) + 1)", ("O1", "r_c"): "C", ("O1", "r_kh"): "KH", ("O1", "r_kw"): "KW"}
    text = nest(src, "fun", [(2, 3, 4, 9, 8), (3, 4, 5, 3, 3)], sym)
    lines = text.strip().split("\n")
    # init nest: LHS indices in declaration order
    assert lines[0] == "for (int O1_s0_n = 0; O1_s0_n < N; O1_s0_n++) {"
    assert lines[4].strip() == "for (int O1_s0_w = 0; O1_s0_w < ((W - KW) + 1); O1_s0_w++) {"
    assert lines[5].strip() == "O1[O1_s0_n][O1_s0_g][O1_s0_f][O1_s0_h][O1_s0_w] = 0.000000f;"
    # update nest: LHS indices outermost, reduction indices innermost in first-appearance order
    order = [re.match(r"\s*for \(int O1_s1_(\w+) =", l).group(1) for l in lines if "O1_s1_" in l and l.strip().startswith("for")]
    assert order == ["n", "g", "f", "h", "w", "r_c", "r_kh", "r_kw"]
    body = [l.strip() for l in lines if l.strip().startswith("O1[O1_s1_n]")][0]
    assert body == ("O1[O1_s1_n][O1_s1_g][O1_s1_f][O1_s1_h][O1_s1_w] = (O1[O1_s1_n][O1_s1_g][O1_s1_f][O1_s1_h][O1_s1_w] + "
                    "(I1[O1_s1_n][O1_s1_g][O1_s1_r_c][(O1_s1_h + O1_s1_r_kh)][(O1_s1_w + O1_s1_r_kw)]*"
                    "W1[O1_s1_g][O1_s1_r_c][O1_s1_f][O1_s1_r_kh][O1_s1_r_kw]));")


def test_loop_nest_copy_and_matmul_golden():
    copy = "def fun(float(P0, P1, P2) I) -> (O) { O(i0, i1, i2) = I(i0, i1, i2) }"
    sym = {("O", "i0"): "P0", ("O", "i1"): "P1", ("O", "i2"): "P2"}
    assert nest(copy, "fun", [(2, 3, 4)], sym).split("\n")[:4] == [
        "for (int O_s0_i0 = 0; O_s0_i0 < P0; O_s0_i0++) {",
        "  for (int O_s0_i1 = 0; O_s0_i1 < P1; O_s0_i1++) {",
        "    for (int O_s0_i2 = 0; O_s0_i2 < P2; O_s0_i2++) {",
        "      O[O_s0_i0][O_s0_i1][O_s0_i2] = I[O_s0_i0][O_s0_i1][O_s0_i2];"]
    mm = "def fun(float(N, K) A, float(K, M) B) -> (O) { O(i, j) +=! A(i, k) * B(k, j) }"
    text = nest(mm, "fun", [(3, 4), (4, 5)], {("O", "i"): "N", ("O", "j"): "M", ("O", "k"): "K"})
    assert "      O[O_s1_i][O_s1_j] = (O[O_s1_i][O_s1_j] + (A[O_s1_i][O_s1_k]*B[O_s1_k][O_s1_j]));" in text.split("\n")


def rng(seed=7):
    return np.random.Generator(np.random.Philox(seed))


def test_batch_matmul_vs_bmm():
    g = rng()
    X, Y = g.standard_normal((5, 26, 72), dtype=np.float32), g.standard_normal((5, 72, 26), dtype=np.float32)
    (Z,) = tc_oracle.run(W.BATCH_MATMUL, "batch_matmul", [X, Y])
    ref = torch.bmm(torch.from_numpy(X).double(), torch.from_numpy(Y).double()).numpy()
    assert np.abs(Z - ref).max() <= W.tolerance(72, ref)


def test_group_convolution_vs_conv2d():
    g = rng(8)
    N, G, C, F, H, Wd, K = 2, 4, 3, 5, 9, 8, 3
    I = g.standard_normal((N, G, C, H, Wd), dtype=np.float32)
    Wt = g.standard_normal((G, F, C, K, K), dtype=np.float32)
    B = g.standard_normal((G, F), dtype=np.float32)
    (O,) = tc_oracle.run(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B])
    ref = torch.conv2d(torch.from_numpy(I).double().reshape(N, G * C, H, Wd),
                       torch.from_numpy(Wt).double().reshape(G * F, C, K, K),
                       torch.from_numpy(B).double().reshape(G * F), groups=G).reshape(N, G, F, H - 2, Wd - 2).numpy()
    assert O.shape == ref.shape
    assert np.abs(O - ref).max() <= W.tolerance(C * K * K, ref)


def test_tensordot_config1_vs_einsum():
    ins = W.make_inputs("c1_tensordot_small")
    (O,) = tc_oracle.run(W.TENSORDOT, "tensordot", ins)
    ref = torch.einsum("nachw,ncbhw->nabhw", torch.from_numpy(ins[0]).double(), torch.from_numpy(ins[1]).double()).numpy()
    assert O.shape == (16, 8, 2, 17, 25)
    assert np.abs(O - ref).max() <= W.tolerance(16, ref)


def test_moments_vs_mean_var():
    X = rng(9).standard_normal((16, 4096), dtype=np.float32) + 3.0
    mean, var = tc_oracle.run(W.MOMENTS, "moments", [X])
    Xd = torch.from_numpy(X).double()
    assert np.abs(mean - Xd.mean(1).numpy()).max() <= W.tolerance(4096, mean)
    assert np.abs(var - Xd.var(1, unbiased=False).numpy()).max() <= W.tolerance(4096, var)


def test_brute_force_float64_on_tiny_shapes():
    g = rng(10)
    I = g.standard_normal((1, 2, 2, 4, 4), dtype=np.float32)
    Wt = g.standard_normal((2, 2, 2, 3, 3), dtype=np.float32)
    B = g.standard_normal((2, 2), dtype=np.float32)
    (fast,) = tc_oracle.run(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B])
    (slow,) = tc_oracle.run_python(W.GROUP_CONVOLUTION, "group_convolution", [I, Wt, B], acc_dtype=np.float64)
    assert np.abs(fast - slow).max() <= 1e-5


def test_integer_inputs_are_exact_and_ones_count_the_reduction():
    g = rng(11)
    X = g.integers(-3, 4, size=(3, 6, 7)).astype(np.float32)
    Y = g.integers(-3, 4, size=(3, 7, 5)).astype(np.float32)
    (Z,) = tc_oracle.run(W.BATCH_MATMUL, "batch_matmul", [X, Y])
    assert np.array_equal(Z, np.einsum("bnm,bmk->bnk", X.astype(np.int64), Y.astype(np.int64)).astype(np.float32))
    ones = [np.ones((2, 3, 5, 4, 4), np.float32), np.ones((2, 5, 2, 4, 4), np.float32)]
    (O,) = tc_oracle.run(W.TENSORDOT, "tensordot", ones)
    assert np.all(O == 5.0)


def test_reduction_operators_and_identities():
    X = rng(12).standard_normal((4, 9), dtype=np.float32)
    src = """
def f(float(M, N) X) -> (mx, mn, pr, cnt) {
    mx(m) max=! X(m, n)
    mn(m) min=! X(m, n)
    pr(m) *=! X(m, n)
    cnt(m) +=! (X(m, n) > 0.0) ? 1.0 : 0.0
}
"""
    X[1] = -np.abs(X[1]) - 1.0      # an all-negative row: max=! must start below every value, not at 0
    X[2] = np.abs(X[2]) + 1.0       # an all-positive row: min=! must start above every value
    mx, mn, pr, cnt = tc_oracle.run(src, "f", [X])
    assert np.array_equal(mx, X.max(1)) and np.array_equal(mn, X.min(1))
    assert mx[1] < 0 and mn[2] > 0
    assert np.allclose(pr, X.astype(np.float64).prod(1), rtol=1e-5)
    assert np.array_equal(cnt, (X > 0).sum(1).astype(np.float32))


def test_non_initialising_reduction_keeps_prior_values():
    src = "def f(float(M, N) X) -> (s) { s(m) += X(m, n) }"
    X = np.ones((3, 5), np.float32)
    prior = np.array([10, 20, 30], np.float32)
    (s,) = tc_oracle.run(src, "f", [X], outputs=[prior.copy()])
    assert np.array_equal(s, prior + 5)


def test_int_literal_division_is_float_when_operand_is_float():
    # mean(m) +=! X(m,n)/N divides a float by an int32 size promoted to float
    X = np.full((2, 8), 3.0, np.float32)
    mean, var = tc_oracle.run(W.MOMENTS, "moments", [X])
    assert np.all(mean == 3.0) and np.all(var == 0.0)


def test_python_interpreter_agrees_with_compiled_nest():
    X = rng(13).standard_normal((2, 10), dtype=np.float32)
    a = tc_oracle.run(W.MOMENTS, "moments", [X])
    b = tc_oracle.run_python(W.MOMENTS, "moments", [X])
    for x, y in zip(a, b):
        assert np.allclose(x, y, atol=1e-6)


def test_storage_of_an_output_starts_at_its_inferred_lower_bound():
    """Shifts of test/test_inference.cc:158-186 executed: the point min + k is element k, so a
    shifted copy returns the input itself, and a reader of the shifted tensor sees its points."""
    I = rng(14).standard_normal(7, dtype=np.float32)
    for stmt in ("O(i) = I(i - 1)", "O(i) = I(i + 5)"):
        src = "def fun(float(I_0) I) -> (O) { %s }" % stmt
        for runner in (tc_oracle.run, tc_oracle.run_python):
            (O,) = runner(src, "fun", [I])
            assert np.array_equal(O, I)
    src = """def f(float(N, M) A) -> (O, P) {
        O(i, j) = A(i, j) * 2.0 where i in 3:N, j in 1:5
        P(i) +=! O(i, j) + A(i - 3, j) }"""
    A = rng(15).integers(-9, 10, size=(12, 7)).astype(np.float32)
    for runner in (tc_oracle.run, tc_oracle.run_python):
        O, P = runner(src, "f", [A])
        assert np.array_equal(O, 2 * A[3:, 1:5])
        assert np.array_equal(P, (2 * A[3:, 1:5] + A[:9, 1:5]).sum(1))


def test_half_is_rounded_after_every_operation():
    """float16 nests are compiled by clang without excess precision: a product is rounded to half
    before it is added, sums accumulate in half."""
    src = "def f(float16(N) a, float16(N) b, float16(N) c) -> (o, s, t) { o(i) = a(i) * b(i) + c(i)\n s(k) +=! a(i) where k in 0:1\n t(k) +=! float(a(i)) where k in 0:1 }"
    a = np.array([1.0009765625, 3.0, 2049.0 - 1.0], np.float16)      # 1 + 2^-10, 3, 2048
    b = np.array([1.0009765625, 0.5, 1.0], np.float16)
    c = np.array([-1.0, 0.25, 1.0], np.float16)
    o, s, t = tc_oracle.run(src, "f", [a, b, c])
    assert o.dtype == np.float16 and s.dtype == np.float16 and t.dtype == np.float32
    # (1 + 2^-10)^2 = 1 + 2^-9 + 2^-20 rounds to 1 + 2^-9 before the subtraction; 2048 + 1 rounds to 2048
    assert np.array_equal(o, np.array([2.0 ** -9, 1.75, 2048.0], np.float16))
    half_sum = np.float16(0)
    for v in a:
        half_sum = np.float16(half_sum + v)
    assert s[0] == half_sum and t[0] == np.float32(a.astype(np.float32).sum())
