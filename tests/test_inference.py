"""Range inference known answers of the reference (test/test_inference.cc:70-540), evaluated at
concrete sizes, for BOTH the oracle and the C++ front end.  The reference prints symbolic
extents; here each expected formula is a Python lambda of the sizes."""
import pytest

import tensorcomprehensions_amd as tc
from oracle import tc_oracle


def cpp_extents(src, entry, shapes):
    return [list(s) for _, s, _ in tc.infer_output_tensor_info(src, entry, [tc.ShapeOnly(s) for s in shapes])]


def oracle_mins_extents(src, entry, shapes):
    an = tc_oracle.analyze(src, entry, shapes)
    return [list(an.tensors[o].mins) for o in an.outputs], [list(an.tensors[o].extents) for o in an.outputs]


# (tc, entry, input shapes, expected mins, expected extents)
def cases():
    I0, I1, I2, I3 = 7, 9, 5, 11
    yield ("def fun(float(I_0) I) -> (O) { O(i) = I(i) }", "fun", [(I0,)], [[0]], [[I0]])
    yield ("def fun(float(I_0, I_1) I) -> (O) { O(i, j) = I(i, j) }", "fun", [(I0, I1)], [[0, 0]], [[I0, I1]])
    yield ("def fun(float(I_0, I_1) I) -> (O) { O(i, j) = I(j, i) }", "fun", [(I0, I1)], [[0, 0]], [[I1, I0]])
    yield ("def fun(float(I_0, I_1, I_2, I_3) I) -> (O) { O(i, j, l, k) = I(j, i, k, l) }", "fun",
           [(I0, I1, I2, I3)], [[0, 0, 0, 0]], [[I1, I0, I3, I2]])
    for n in (1, 122, 123, 124, 1000):
        yield ("def fun(float(I_0) I) -> (O) { O(i) = I(123 * i) }", "fun", [(n,)], [[0]], [[(n + 122) // 123]])
    yield ("def fun(float(I_0) I) -> (O) { O(i) = I(i - 1) }", "fun", [(I0,)], [[1]], [[I0]])
    yield ("def fun(float(I_0) I) -> (O) { O(i) = I(i + 5) }", "fun", [(I0,)], [[-5]], [[I0]])
    N, C, H, W, M, KH, KW = 2, 3, 12, 13, 4, 3, 5
    conv = """def convolution(float(N,C,H,W) I, float(M,C,KH,KW) W1, float(M) B) -> (tmp, O) {
        tmp(n, m, h, w) +=! I(n, c, h + kh, w + kw) * W1(m, c, kh, kw)
        O(n, m, h, w) +=! tmp(n, m, h, w) + B(m) }"""
    e = [N, M, H - KH + 1, W - KW + 1]
    yield (conv, "convolution", [(N, C, H, W), (M, C, KH, KW), (M,)], [[0] * 4, [0] * 4], [e, e])
    # the symbolic answer is non-empty only when d_O is at least as large as I
    OH, OW = H + 2, W + 1
    grad = """def convolutionGrad(float(N,C,H,W) I, float(M,C,KH,KW) W1, float(N,M,OH,OW) d_O) -> (d_I, d_W1, d_B) {
        d_I(n, c, h, w) +=! d_O(n, m, h - kh, w - kw) * W1(m, c, kh, kw)
        d_W1(m, c, kh, kw) +=! d_O(n, m, h - kh, w - kw) * I(n, c, h, w)
        d_B(m) +=! d_O(n, m, h, w) }"""
    yield (grad, "convolutionGrad", [(N, C, H, W), (M, C, KH, KW), (N, M, OH, OW)],
           [[0, 0, KH - 1, KW - 1], [0, 0, H - OH, W - OW], [0]],
           [[N, C, OH - KH + 1, OW - KW + 1], [M, C, OH - H + 1, OW - W + 1], [M]])
    padded = """def convolution(float(N,C,H,W) I, float(M,C,KH,KW) W1, float(M) B) -> (pad, tmp) {
        pad(n, c, h, w)  = I(n, c, h - 2 - 3, w - 3 - 4)
        tmp(n, m, h, w) +=! pad(n, c, 2 * h + kh, 3 * w + kw) * W1(m, c, kh, kw) }"""
    for (H2, W2) in ((12, 13), (20, 31), (9, 8)):
        yield (padded, "convolution", [(N, C, H2, W2), (M, C, KH, KW), (M,)],
               [[0, 0, 5, 7], [0, 0, 3, 3]], [[N, C, H2, W2], [N, M, (H2 - KH + 1) // 2, (W2 - KW + 1) // 3]])
    weird = """def fun(float(B,IP,H,W) input, float(OP,IP,KH,KW) weight) -> (output) {
      output(b, op, h, w) +=! input(b, ip, 2 * h + 3 * w + kh, 2 * w + kw) * weight(op, ip, kh, kw) }"""
    for (H2, W2) in ((40, 13), (64, 21)):
        yield (weird, "fun", [(2, 3, H2, W2), (4, 3, KH, KW)], [[0] * 4],
               [[2, 4, ((H2 - KH) - ((W2 - KW) // 2) * 3) // 2 + 1, (W2 - KW) // 2 + 1]])
    yield ("def fun(float(I_0, I_1, I_2) I) -> (O) { O(i) +=! I(j, i + j, k) }", "fun", [(4, 9, 3)], [[0]], [[9 - 4 + 1]])
    A, B, Cc = (6, 7, 8), (5, 9, 4), (3, 2, 6)
    tcf = """def fun(float(A_0, A_1, A_2) A, float(B_0, B_1, B_2) B, float(C_0, C_1, C_2) C) -> (O2, O3) {
      O2(j, k, l) +=! B(j, k, l) + A(i, j, k)
      O3(k, l, m) +=! C(k, l, m) + O2(j, k, l) }"""
    yield (tcf, "fun", [A, B, Cc], [[0] * 3, [0] * 3],
           [[min(B[0], A[1]), min(B[1], A[2]), B[2]], [min(Cc[0], min(B[1], A[2])), min(Cc[1], B[2]), Cc[2]]])
    tcg = """def fun(float(A_0, A_1, A_2) A, float(B_0, B_1, B_2) B, float(C_0, C_1, C_2) C) -> (O1, O2, O3) {
      O1(i, j) +=! A(i, j, k)
      O2(j, k, l) +=! B(j, k, l) + O1(i, j)
      O3(k, l, m) +=! C(k, l, m) + O2(j, k, l) }"""
    yield (tcg, "fun", [A, B, Cc], [[0] * 2, [0] * 3, [0] * 3],
           [[A[0], A[1]], [min(B[0], A[1]), B[1], B[2]], [min(Cc[0], B[1]), min(Cc[1], B[2]), Cc[2]]])
    yield ("def fun(float(N, M) I) -> (O) { O(i, j) = I(i, j) where i in 3:N-1 }", "fun", [(10, 6)], [[3, 0]], [[10 - 4, 6]])
    for (n, m) in ((30, 40), (15, 25), (12, 25), (25, 17)):
        yield ("def fun(float(N, M) I) -> (O) { O(i, j) = I(10 + i - j, i + j) where i in 0:10 }", "fun", [(n, m)],
               [[0, 20 - min(n, 20)]], [[10, (min(m - 10, 10) + min(n, 20)) - 19]])
    yield ("def fun(float(10, 19, 10) I) -> (O) { O(i, j) = I(i, i + j, j) }", "fun", [(10, 19, 10)], [[0, 0]], [[10, 10]])
    yield ("def fun() -> (O) { O(i, j) = 3 where i in 4:8, j in 3:20 }", "fun", [], [[4, 3]], [[4, 17]])
    yield ("def fun() -> (O) { O(i, j) = 3 where i in 8:4, j in 3:20 }", "fun", [], [[8, 3]], [[-4, 17]])


@pytest.mark.parametrize("src,entry,shapes,mins,extents", list(cases()))
def test_inferred_ranges(src, entry, shapes, mins, extents):
    omins, oext = oracle_mins_extents(src, entry, shapes)
    assert omins == mins
    assert oext == extents
    assert cpp_extents(src, entry, shapes) == extents


# ill-formed or ambiguous definitions: both front ends must refuse (warnings are errors here,
# as in the reference's test fixture, test/test_inference.cc:29-31)
BAD = [
    ("def fun(float(I_0, I_1, I_2, I_3, I_4) I) -> (O) { O(i, j, k, l, m) = I(j, i, k, i, l) }", [(3, 3, 3, 3, 3)]),
    ("def fun(float(I_0, I_1, I_2) A) -> (O) { O(i) +=! A(i + j, i + j, i + j) }", [(4, 4, 4)]),
    ("def fun(float(I_0, I_1, I_2) I) -> (O) { O(i) +=! I(i, i + j, j) }", [(4, 5, 4)]),
    ("def fun(float(I_0, I_1, I_2, I_3, I_4) I) -> (O) { O(i) +=! I(i, j, i, k, 2 * i + j) }", [(4, 4, 4, 4, 4)]),
    ("def fun(float(I_0, I_1, I_2, I_3, I_4) I) -> (O) { O(i) +=! I(j, j + 1, i, i + 3, 2 * i + j + 0) }", [(4, 5, 4, 7, 4)]),
    ("def fun(float(N, M) I) -> (O) { O(i, j) = I(10 + i - j, i + j) }", [(30, 40)]),
    ("def fun(float(N, NM, M) I) -> (O) { O(i, j) = I(i, i + j, j) }", [(10, 12, 10)]),
    ("def fun() -> (O) { O(i, j) = 3 }", []),
    ("def fun(float(N) size) -> (O) { O(i, j) = 3 where i in 0:size(j), j in 0:size(i) }", [(5,)]),
]


@pytest.mark.parametrize("src,shapes", BAD)
def test_rejected_definitions(src, shapes):
    with pytest.raises(tc_oracle.TcError):
        an = tc_oracle.analyze(src, "fun", shapes)
        if an.warnings:
            raise tc_oracle.TcError(an.warnings[0])
    tc.set_compiler_options(emit_warnings=False, throw_warnings=True)
    try:
        with pytest.raises(tc.TcError):
            cpp_extents(src, "fun", shapes)
    finally:
        tc.set_compiler_options(True, False)


def test_size_mismatch_and_constant_dims():
    mm = "def mm(float(M,K) A, float(K,N) B) -> (C) { C(m,n) +=! A(m,r_k) * B(r_k,n) }"
    with pytest.raises(tc.TcError) as e:
        cpp_extents(mm, "mm", [(3, 4), (5, 6)])
    assert "Mismatched sizes for dimension K" in str(e.value)
    with pytest.raises(tc_oracle.TcError):
        tc_oracle.analyze(mm, "mm", [(3, 4), (5, 6)])
    const = "def f(float(10, 19) I) -> (O) { O(i) +=! I(i, j) }"
    with pytest.raises(tc.TcError) as e:
        cpp_extents(const, "f", [(10, 18)])
    assert "Constant dimension expected size 19 but found 18" in str(e.value)
    with pytest.raises(tc.TcError) as e:
        cpp_extents(mm, "mm", [(3, 4)])
    assert "expected 2 inputs" in str(e.value)
    with pytest.raises(tc.TcError) as e:
        cpp_extents(mm, "mm", [(3, 4, 1), (4, 6)])
    assert "expected a tensor with 2 dimensions but found 3 dimensions" in str(e.value)
