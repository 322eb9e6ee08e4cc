"""Size-parametric range inference (csrc/tc/core/symbolic_ranges.cc) against the symbolic known
answers the reference's own tests hold (test/test_inference.cc:70-540, extracted as data by
tests/golden/make_inference_fixtures.py) and against the concrete inference of the compile path.

The reference prints Halide-simplified expressions; two formulas are the same when they agree for
every assignment of the sizes, which is what is checked (on random sizes, small ones included)."""
import json
import os
import random
import re

import pytest

import tensorcomprehensions_amd as tc
from tensorcomprehensions_amd.symbolic import evaluate
from oracle import tc_oracle
from tests import benchmark_tcs as B
from tests import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, "golden", "inference", "known_answers.json")))


def parse_reference_dump(text):
    """{'mins': {tensor: [expr]}, 'extents': {...}} of a 'mins:/extents:' text; Halide prints
    integer division as '/', which rounds toward minus infinity like Python's '//'."""
    out, section = {"mins": {}, "extents": {}}, None
    for line in text.splitlines():
        if line in ("mins:", "extents:"):
            section = line[:-1]
        elif "@[" in line:
            name, rest = line.split("@[", 1)
            out[section][name] = [d.strip().replace("/", "//") for d in rest.rstrip("]").split(";") if d.strip()]
    return out


@pytest.mark.parametrize("case", GOLDEN, ids=[c["name"] for c in GOLDEN])
def test_symbolic_bounds_equal_the_references_known_answers(case):
    ours = tc.infer_ranges(case["tc"])
    ref = parse_reference_dump(case["expected"])
    mine = {"mins": {}, "extents": {}}
    for group in (ours.inputs, ours.outputs):
        for name, (mins, ext) in group.items():
            mine["mins"][name], mine["extents"][name] = mins, ext
    assert list(mine["mins"]) == list(ref["mins"]), "tensors in the reference's order"
    params = sorted(set(re.findall(r"[A-Za-z_]\w*", " ".join(sum(ref["extents"].values(), [])))) - {"min", "max"})
    rng = random.Random(7)
    for trial in range(60):
        sizes = {p: rng.randint(1, 12) if trial % 3 == 0 else rng.randint(1, 64) for p in params}
        for kind in ("mins", "extents"):
            for name, exprs in ref[kind].items():
                assert len(exprs) == len(mine[kind][name]), (name, kind)
                for d, (theirs, here) in enumerate(zip(exprs, mine[kind][name])):
                    assert evaluate(theirs, sizes) == evaluate(here, sizes), (name, kind, d, theirs, here, sizes)


def concrete_cases():
    for name, (src, entry, shapes, _, _) in W.CONFIGS.items():
        yield name, src, [tuple(s) for s in shapes]
    for name, (src, entry, specs, _) in B.CASES.items():
        shapes = [tuple(a.shape) for a in B.make_inputs(name)]
        yield name, src, shapes
    conv = """def convolution(float(N,C,H,W) I, float(M,C,KH,KW) W1, float(M) B) -> (tmp, O) {
        tmp(n, m, h, w) +=! I(n, c, h + kh, w + kw) * W1(m, c, kh, kw)
        O(n, m, h, w) +=! tmp(n, m, h, w) + B(m) }"""
    yield "conv", conv, [(2, 3, 12, 13), (4, 3, 3, 5), (4,)]
    weird = """def fun(float(B,IP,H,W) input, float(OP,IP,KH,KW) weight) -> (output) {
      output(b, op, h, w) +=! input(b, ip, 2 * h + 3 * w + kh, 2 * w + kw) * weight(op, ip, kh, kw) }"""
    for hw in ((40, 13), (64, 21), (33, 17)):
        yield f"weird{hw}", weird, [(2, 3) + hw, (4, 3, 3, 5)]
    yield "shift", "def fun(float(I_0) I) -> (O) { O(i) = I(i - 1) }", [(7,)]
    yield "stride", "def fun(float(I_0) I) -> (O) { O(i) = I(123 * i) }", [(1000,)]
    yield "rotate", "def fun(float(N, M) I) -> (O) { O(i, j) = I(10 + i - j, i + j) where i in 0:10 }", [(25, 40)]
    yield "let", "def fun(float(N, M) I) -> (O) { O(i, j) = I(k, j) where k = i + 2 }", [(9, 5)]
    yield "sized_where", "def fun(float(N, M) I) -> (O) { O(i, j) = I(i, j) where i in 3:N-1 }", [(9, 5)]


@pytest.mark.parametrize("name,src,shapes", list(concrete_cases()), ids=[c[0] for c in concrete_cases()])
def test_specialised_symbolic_bounds_equal_the_concrete_inference(name, src, shapes):
    """Late specialisation: the formulas evaluated at the sizes of a call give the bounds the compile
    path infers on those sizes (extents from the C++ front end, lower bounds from the oracle)."""
    entry = re.search(r"def\s+(\w+)", src).group(1)
    sym = tc.infer_ranges(src)
    bounds = sym.output_bounds(shapes)
    extents = [list(s) for _, s, _ in tc.infer_output_tensor_info(src, entry, [tc.ShapeOnly(s) for s in shapes])]
    assert [e for _, e in bounds] == extents
    an = tc_oracle.analyze(src, entry, shapes)
    assert [m for m, _ in bounds] == [list(an.tensors[o].mins) for o in an.outputs]
    assert [e for _, e in bounds] == [list(an.tensors[o].extents) for o in an.outputs]


def test_statement_ranges_and_parameters_are_reported():
    sym = tc.infer_ranges(W.CONFIGS["c4_group_convolution"][0])
    assert sym.parameters[:3] == ["N", "G", "C"]
    tensor, variables = sym.statements[0]
    ranges = {v: (lo, hi) for v, lo, hi in variables}
    assert tensor == "O" and ranges["h"] == ("0", "H - KH") and ranges["kh"] == ("0", "KH - 1")


def test_what_the_concrete_inference_refuses_for_every_size_is_refused_here():
    with pytest.raises(tc.TcError, match="was not solved in range inference"):
        tc.infer_ranges("def fun() -> (O) { O(i, j) = 3 }")
    with pytest.raises(tc.TcError):
        tc.infer_ranges("def fun(float(N) size) -> (O) { O(i, j) = 3 where i in 0:size(j), j in 0:size(i) }")
    with pytest.raises(ValueError, match="mismatched sizes"):
        tc.infer_ranges("def mm(float(M,K) A, float(K,N) B) -> (C) { C(m,n) +=! A(m,r_k) * B(r_k,n) }").sizes_from([(3, 4), (5, 6)])
