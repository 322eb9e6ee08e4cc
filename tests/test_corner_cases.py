"""The reference's corner cases (test/cuda/test_corner_cases.cc:82-345): short programs that must
either fail with a recognisable message or run.  Failures are raised while compiling, so they are
checked without a GPU; the ones that must run are GPU tests and compare values as the reference
does."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc


def F(*shape):
    return tc.ShapeOnly(shape, "float32")


def I(*shape):
    return tc.ShapeOnly(shape, "int32")


FAILS = {
    "E1": ("expected (", " def f{} {}", []),
    "E7": ("expected 2 inputs", "def f(float a, float c) -> (b) { b(i) = a where i in 0:10 }", [F()]),
    "E8": ("expected type int32", "def f(int32 a) -> (b) { b(i) = a where i in 0:10 }", [F()]),
    "E9": ("expected a tensor with 0", "def f(int32 a) -> (b) { b(i) = a where i in 0:10 }", [I(1, 2)]),
    "E11": ("expected integral type", "def f(int32(N) a) -> (b) { b(i) = a(i + .5) }", [I(10)]),
    "E12": ("tensor accesses cannot be used in this context",
            "def f(int32 a, float(N) b) -> (c) { c(i) += b(i + j) where j in 0:a, i in 0:10 }", [I(), F(12)]),
    "E13": ("tensor accesses cannot be used in this context",
            "def f(int32 a, float(N) b) -> (c) { c(i) += b(i + j) where j in 0:a }", [I(), F(12)]),
    "E19": ("undefined variable", "def f(float(1) a) -> (b) { b(i) = 2*foo where foo = a(i), foo in 1:2 }", [F(1)]),
    "E20": ("Temporaries tensors", "def f(float(1) a) -> (b) { c(i) = a(i) b(i) = c(i)  }", [F(1)]),
}


@pytest.mark.parametrize("case", sorted(FAILS))
def test_fails_with_the_expected_fragment(case):
    fragment, src, inputs = FAILS[case]
    with pytest.raises(tc.TcError) as e:
        tc.compile(src, "f", inputs, "naive")
    assert fragment in str(e.value), str(e.value)


def run(src, *inputs):
    ins = [torch.as_tensor(x).cuda() for x in inputs]
    ex = tc.compile(src, "f", ins, "naive")
    outs = tc.prepare_outputs(src, "f", ins)
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu() for o in outs]


@pytest.mark.gpu
def test_degenerate_shapes_run():
    a = torch.tensor([3.5])
    assert run("def f(float(1) a) -> (b) { b(i) = a(i) }", a)[0].tolist() == [3.5]                      # E2
    s = torch.tensor(2.25)
    (b,) = run("def f(float a) -> (b) { b = a }", s)                                                      # E4
    assert b.dim() == 0 and b.item() == 2.25
    assert run("def f(float a) -> (b) { b(i) = a where i in 0:10 }", s)[0].tolist() == [2.25] * 10        # E6
    (b,) = run("def f(int32 a) -> (b) { b(i) = a where i in 0:10 }", torch.tensor(7, dtype=torch.int32))  # E10
    assert b.dtype == torch.int32 and b.tolist() == [7] * 10


@pytest.mark.gpu
def test_wrong_output_rank_is_refused_at_run_time():
    src = "def f(float(1) a) -> (b) { b(i) = a(i) }"                                                     # E25
    a = torch.ones(1).cuda()
    ex = tc.compile(src, "f", [a], "naive")
    with pytest.raises(tc.TcError) as e:
        tc.run(ex, [a], [torch.ones(1, 1).cuda()])
    assert "expected 1 dimensions but found tensor with 2 dimensions" in str(e.value)


@pytest.mark.gpu
@pytest.mark.parametrize("op", ["<=", ">=", "==", "!=", "<", ">"])
def test_comparisons(op):                                                                                # E15
    for x, y in ((0.25, 0.75), (0.75, 0.25), (0.5, 0.5)):
        (c,) = run(f"def f(float a, float b) -> (c) {{ c(i) = float(a {op} b) where i in 0:1 }}", torch.tensor(x), torch.tensor(y))
        assert c.item() == float(eval(f"{x} {op} {y}"))


@pytest.mark.gpu
@pytest.mark.parametrize("op,py", [("||", "or"), ("&&", "and")])
def test_boolean_operators_and_precedence(op, py):                                                       # E16
    for x in (0.25, 0.75):
        for y in (0.25, 0.75):
            (c,) = run(f"def f(float a, float b) -> (c) {{ c(i) = float(!(a < .5) {op} b > .5) where i in 0:1 }}",
                       torch.tensor(x), torch.tensor(y))
            assert c.item() == float(eval(f"(not ({x} < .5)) {py} ({y} > .5)"))


@pytest.mark.gpu
def test_exists_let_min_max_and_newlines():
    a, b, c = torch.tensor([0.3]), torch.tensor([0.9]), torch.tensor([0.6])
    assert run("def f(float(1) a) -> (b) { b(i) = 4.0 where exists a(i) }", a)[0].item() == 4.0           # E17
    assert run("def f(float(1) a) -> (b) { b(i) = 2*foo where foo = a(i) }", a)[0].item() == pytest.approx(0.6)  # E18
    assert run("def f(float(1) a, float(1) b) -> (c) { c(i) = max(a(i), b(i)) }", a, b)[0].item() == pytest.approx(0.9)  # E21
    assert run("def f(float(1) a, float(1) b) -> (c) { c(i) = min(a(i), b(i)) }", a, b)[0].item() == pytest.approx(0.3)  # E22
    src = "def f(float(1) a, float(1) b, float(1) c) -> (d) { d(i) = min(a(i), max(b(i), c(i))) }"      # E23
    assert run(src, a, b, c)[0].item() == pytest.approx(min(0.3, max(0.9, 0.6)))
    ragged = """

def f(float(1)
a, float(1
) b, float
(1) c) -> (d) { d(
i)
 =

 min(
a(i), max(
b(i), c(
i)))

d(i) = d(i) + max(b(i),

c(
i))

}
"""
    assert run(ragged, a, b, c)[0].item() == pytest.approx(min(0.3, max(0.9, 0.6)) + max(0.9, 0.6))      # E24


@pytest.mark.gpu
def test_integer_modulo():                                                                               # E26
    (r,) = run("def f(int32 a, int32 b) -> (c) { c(i) = int32(a % b) where i in 0:1 }",
               torch.tensor(17, dtype=torch.int32), torch.tensor(5, dtype=torch.int32))
    assert r.dtype == torch.int32 and r.item() == 17 % 5


SHRINKING = """def f(float(K, P, M, P) A) -> (O) {
    O(i) = float(i + 3) where i in 0:16
    O(i) min= A(i, j, i, i)
}"""


def test_a_tensor_takes_the_bounds_of_its_last_definition_in_every_statement():
    """tc2halide.cc:676-693 clobbers a tensor's bounds with those of its last definition and applies
    them to all its stages: `O` is inferred as 16 elements by the first statement and as one by the
    second (`i` also indexes a dimension of size 1), so it has one element and the first statement
    writes one element, not sixteen."""
    from oracle import tc_oracle
    assert [s for _, s, _ in tc.infer_output_tensor_info(SHRINKING, "f", [F(16, 70, 1, 70)])] == [(1,)]
    assert tc_oracle.infer_output_shapes(SHRINKING, "f", [(16, 70, 1, 70)]) == [("O", "float", [1])]
    src, launches = tc.map_only(SHRINKING, "f", [F(16, 70, 1, 70)], "naive;outerScheduleFusionStrategy=Min")
    assert all(block == (1, 1, 1) for _, block in launches)
    A = np.full((16, 70, 1, 70), 7.0, np.float32)
    (o,) = tc_oracle.run(SHRINKING, "f", [A])
    assert o.tolist() == [3.0]


@pytest.mark.parametrize("text,shapes", [
    ("def f(float(N) A) -> (O) { O(i) = A(i) where i in 2:2 }", [(5,)]),
    ("def f(float(N) A) -> (O) { O(i) = A(i) where i in 4:1 }", [(5,)]),
    # empty for one statement of a tensor that a later statement defines over five elements
    ("def f(float(N, K) A, float(N, P) B) -> (O) { O(i) = float(1.5) where i in 0:0\n O(i) += A(i, i) + B(i, j) }", [(5, 6), (5, 7)]),
    ("def f(float(N) A) -> (O) { O(i) +=! A(i + j) where j in 3:3 }", [(5,)]),
])
def test_a_range_given_empty_is_refused(text, shapes):
    """`where i in a:b` with b <= a: nothing would run over it (a loop variable without points used
    to reach the mapper and divide by its tile size of zero).  Range inference itself accepts it and
    reports a negative extent, as the reference's does (test/test_inference.cc:498-511, a known
    answer of tests/test_inference.py); mapping, compiling and the oracle's execution refuse it."""
    from oracle import tc_oracle
    with pytest.raises(tc.TcError, match="Empty range for variable"):
        tc.map_only(text, "f", [F(*s) for s in shapes], "naive")
    with pytest.raises(tc.TcError, match="Empty range for variable"):
        tc.compile(text, "f", [F(*s) for s in shapes], "naive")
    with pytest.raises(tc_oracle.TcError, match="Empty range for variable"):
        tc_oracle.run(text, "f", [np.zeros(s, np.float32) for s in shapes])


def test_a_tensor_is_written_with_the_same_number_of_subscripts_by_every_statement():
    """`O(i) = ...` followed by `O(j, i) = ...`: the reference's sema keeps the first definition's
    type and lets the second through (tc/lang/sema.h:566-571; Halide then refuses the update
    definition).  Here the statement is refused by sema and by the oracle: it used to reach the
    code generator, which read past the strides of the one-dimensional tensor."""
    from oracle import tc_oracle
    text = """def f(float(P, M, M) A, float(Q) B) -> (O0, O1) {
        O0(i) max=! tanh(A(i, j, k) + B(l))
        O1(i) = O0(i) * 0.5 + 1
        O1(j, i) = A(i, j, i) * Q }"""
    for call in (lambda: tc.infer_output_tensor_info(text, "f", [F(3, 4, 4), F(5)]),
                 lambda: tc.map_only(text, "f", [F(3, 4, 4), F(5)], "naive")):
        with pytest.raises(tc.TcError, match="O1 was defined with 1 dimensions and is written here with 2"):
            call()
    with pytest.raises(tc_oracle.TcError, match="O1 was defined with 1 dimensions and is written here with 2"):
        tc_oracle.infer_output_shapes(text, "f", [(3, 4, 4), (5,)])
    # fewer subscripts than before, and an annotated output
    with pytest.raises(tc.TcError, match="was defined with 2 dimensions and is written here with 1"):
        tc.map_only("def g(float(N, M) A) -> (O) { O(n, m) = A(n, m)\n O(n) = A(n, 0) }", "g", [F(4, 5)], "naive")


def test_later_statement_cannot_narrow_into_the_tensors_first_type():
    """`O` is int32 by its first definition; accumulating floats into it would be an update
    definition of another type, which the reference's Halide lowering refuses.  The front end and
    the oracle say so in the words used for annotated outputs; with an explicit cast, or a float
    initial value, the program is accepted."""
    from oracle import tc_oracle
    bad = "def f(float(N) A) -> (O) { O(i) = 0 where i in 0:4\n O(i) += A(i) * 1.5 }"
    with pytest.raises(tc.TcError) as e:
        tc.map_only(bad, "f", [F(4)], "naive")
    assert "to narrower type" in str(e.value)
    with pytest.raises(tc_oracle.TcError) as e:
        tc_oracle.infer_output_shapes(bad, "f", [(4,)])
    assert "to narrower type" in str(e.value)
    for good in ("def f(float(N) A) -> (O) { O(i) = 0 where i in 0:4\n O(i) += int32(A(i) * 1.5) }",
                 "def f(float(N) A) -> (O) { O(i) = 0.0 where i in 0:4\n O(i) += A(i) * 1.5 }"):
        tc.map_only(good, "f", [F(4)], "naive")
        tc_oracle.infer_output_shapes(good, "f", [(4,)])


# ------------------------------------------------------------------------------------------------
# tensors a kernel must never be launched on: refused before any launch, so checked without a GPU
# (the reference launches on whatever pointer it is given, tc/core/tc_executor-inl.h:109-145)
# ------------------------------------------------------------------------------------------------
COPY = "def f(float(N) a) -> (b) { b(i) = a(i) }"


def _copy_executor():
    return tc.compile(COPY, "f", [F(8)], "naive")


@pytest.mark.parametrize("entry", ["run", "profile", "call", "autotune"])
def test_host_tensors_are_refused_before_any_launch(entry):
    ex = _copy_executor()
    a, b = torch.zeros(8), torch.zeros(8)
    with pytest.raises(tc.TcError) as e:
        if entry == "run":
            tc.run(ex, [a], [b])
        elif entry == "profile":
            tc.profile(ex, [a], [b])
        elif entry == "call":
            ex(a)
        else:
            tc.autotune(COPY, "f", [a], "naive", outputs=[b], generations=1, pop_size=2)
    assert "not in HIP device memory" in str(e.value), str(e.value)


def test_null_data_pointers_are_refused_before_any_launch():
    ex = _copy_executor()
    with pytest.raises(tc.TcError) as e:
        tc.run(ex, [F(8)], [F(8)])
    assert "null data pointer" in str(e.value), str(e.value)
    with pytest.raises(tc.TcError) as e:
        tc.autotune(COPY, "f", [F(8)], "naive", outputs=[F(8)], generations=1, pop_size=2)
    assert "null data pointer" in str(e.value), str(e.value)
