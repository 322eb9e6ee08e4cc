"""CPU oracle for Tensor Comprehensions semantics.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU, what the reference computes for a TC definition:
parse -> semantic analysis -> forward range inference -> canonical sequential
loop nest.  It exists so that the HIP backend can be checked against an
independent implementation.  Only tests, the smoke check and the cpu_baseline
leg of the benchmark may import it; the product never does.

Reference files followed (paths relative to the reference checkout):
  * grammar / token rules ............ tc/lang/lexer.h:37-92,135-307, tc/lang/parser.h:23-318
  * typing, reduction variables ...... tc/lang/sema.h:129-163 (match_types), :230-240, :498-620
  * range inference .................. tc/core/tc2halide.cc:270-498 (forwardBoundsInference)
  * statement lowering, identities ... tc/core/tc2halide.cc:560-609
  * loop order ....................... tc/core/tc2halide.cc:698-755 (LHS indices outermost in
                                       declaration order, reduction indices innermost in
                                       left-to-right first-appearance order)
  * output shapes .................... tc/core/halide_utils.cc:41-119
  * the sequential CPU path .......... tc/core/polyhedral/cpu/mapped_scop.cc:49-91,
                                       tc/core/polyhedral/codegen_llvm.cc:621-644

The loop nest is emitted as C (same text shape as the golden nests in
test/test_core.cc:93-232), compiled with gcc -O3 without fast-math or FMA
contraction, and called through ctypes on numpy arrays.  A pure-Python
interpreter of the same nest (`run_python`) exists for tiny shapes.  Nests
with float16 tensors (a type the reference's front end refuses, tc/lang/sema.h:62-66,
so nothing of the reference pins them: "parity unpinned", checked against IEEE
half arithmetic in numpy and closed forms instead) are compiled with the ROCm
clang, `-fexcess-precision=16`: every operation is rounded to half.

Pinned by tests/test_oracle_*.py against: the reference's range-inference
known answers (test/test_inference.cc:70-540), its golden loop nests
(test/test_core.cc:93-232), library routines that the reference's own tests use
as ground truth (einsum / bmm / conv2d(groups) / mean,var), float64 brute force
and integer-valued inputs (exact sums).

Known restriction: non-affine subscripts (indirection, %, /) contribute no range
constraint here (the reference drops them with a warning once their variables
are solved, tc2halide.cc:448-465).  The storage of an output starts at its inferred
lower bound (element k of a dimension holds the point min + k).
"""
from __future__ import annotations

import ctypes
import hashlib
import tempfile
import math
import os
import re
import subprocess
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

# ----------------------------------------------------------------------------------------------
# Lexer  (tc/lang/lexer.h:37-92 token table, :206-212 comments, :186-200 numbers via strtod)
# ----------------------------------------------------------------------------------------------
_MULTI = ["+=!", "*=!", "min=!", "max=!", "<=>", "+=", "*=", "min=", "max=", "->", ">=", "<=", "==", "!=", "&&", "||"]
_SINGLE = "+-*/()[]?:,={}><!%"
_SCALAR_TYPES = {
    "bool": ("uint", 1), "uint8": ("uint", 8), "uint16": ("uint", 16), "uint32": ("uint", 32),
    "uint64": ("uint", 64), "int8": ("int", 8), "int16": ("int", 16), "int32": ("int", 32),
    "int64": ("int", 64), "float16": ("float", 16), "float32": ("float", 32), "float64": ("float", 64),
    "float": ("float", 32), "double": ("float", 64),
}
_KEYWORDS = {"min", "max", "where", "def", "in", "exists"} | set(_SCALAR_TYPES)
_NUM_RE = re.compile(r"(?:\d+\.?\d*(?:[eE][+-]?\d+)?|\.\d+(?:[eE][+-]?\d+)?)")
_ID_RE = re.compile(r"[A-Za-z_][A-Za-z_0-9]*")


class TcError(Exception):
    """Counterpart of lang::ErrorReport (tc/lang/error_report.h:23-44)."""


def tokenize(src: str) -> List[Tuple[str, str, int]]:
    toks = []
    i, n = 0, len(src)
    while i < n:
        c = src[i]
        if c.isspace():
            i += 1
            continue
        if c == "#":
            while i < n and src[i] != "\n":
                i += 1
            continue
        m = _NUM_RE.match(src, i)
        if m and m.end() > i:
            toks.append(("number", m.group(0), i))
            i = m.end()
            continue
        # longest match between identifier and operator tokens; keyword tokens such as
        # "min=" beat the identifier "min" (lexer.h:236-262)
        best = None
        for t in _MULTI:
            if src.startswith(t, i) and (best is None or len(t) > len(best)):
                best = t
        m = _ID_RE.match(src, i)
        if m and (best is None or len(m.group(0)) > len(best)):
            word = m.group(0)
            toks.append((word if word in _KEYWORDS else "ident", word, i))
            i = m.end()
            continue
        if best is not None:
            toks.append((best, best, i))
            i += len(best)
            continue
        if c in _SINGLE:
            toks.append((c, c, i))
            i += 1
            continue
        raise TcError(f"expected a valid token but found '{c}' at offset {i}")
    toks.append(("eof", "", n))
    return toks


# ----------------------------------------------------------------------------------------------
# Parser (Pratt; precedences from tc/lang/lexer.h:138-151)
# ----------------------------------------------------------------------------------------------
_BINPREC = {"?": 1, "||": 2, "&&": 3, ">": 4, "<": 4, "<=": 4, ">=": 4, "==": 4, "!=": 4,
            "+": 5, "-": 5, "*": 6, "/": 6, "%": 6}
_UNPREC = 7
_ASSIGN = {"=", "+=", "*=", "min=", "max=", "+=!", "*=!", "min=!", "max=!"}


@dataclass
class Expr:
    kind: str                    # const | ident | apply | access | builtin | bin | un | sel | cast
    op: str = ""                 # operator / name / type
    args: List["Expr"] = field(default_factory=list)
    value: float = 0.0
    type: Optional[str] = None   # filled in by sema: scalar type name


@dataclass
class Param:
    name: str
    scalar: Optional[str]        # None = inferred
    dims: List[object]           # str (size variable) or int


@dataclass
class Stmt:
    lhs: str
    indices: List[str]
    assign: str
    rhs: Expr
    where: List[tuple]
    reduction_vars: List[str] = field(default_factory=list)
    ranges: Dict[str, Tuple[int, int]] = field(default_factory=dict)   # inclusive
    scalar: str = "float"


@dataclass
class Def:
    name: str
    params: List[Param]
    returns: List[Param]
    stmts: List[Stmt]


class _Parser:
    def __init__(self, src: str):
        self.toks = tokenize(src)
        self.p = 0

    @property
    def cur(self):
        return self.toks[self.p]

    def next(self):
        t = self.toks[self.p]
        self.p += 1
        return t

    def accept(self, kind):
        if self.cur[0] == kind:
            return self.next()
        return None

    def expect(self, kind):
        if self.cur[0] != kind:
            raise TcError(f"expected {kind} but found '{self.cur[1] or self.cur[0]}' at offset {self.cur[2]}")
        return self.next()

    def parse_const(self):
        t = self.expect("number")[1]
        ty = "float" if ("." in t or "e" in t) else "int32"       # parser.h:33-40
        return Expr("const", value=float(t), type=ty)

    def parse_base(self):
        k = self.cur[0]
        if k == "number":
            return self.parse_const()
        if k == "(":
            self.next()
            e = self.parse_exp()
            self.expect(")")
            return e
        if k in _SCALAR_TYPES:
            ty = self.next()[0]
            self.expect("(")
            e = self.parse_exp()
            self.expect(")")
            return Expr("cast", op=ty, args=[e])
        if k in ("min", "max"):
            self.next()
            self.expect("(")
            a = self.parse_exp()
            self.expect(",")
            b = self.parse_exp()
            self.expect(")")
            return Expr("bin", op=k, args=[a, b])
        name = self.expect("ident")[1]
        if self.cur[0] == "(":
            return Expr("apply", op=name, args=self.parse_list(self.parse_exp))
        return Expr("ident", op=name)

    def parse_exp(self, prec=0):
        if self.cur[0] in ("-", "!"):
            op = self.next()[0]
            left = Expr("un", op=op, args=[self.parse_exp(_UNPREC)])
        else:
            left = self.parse_base()
        while self.cur[0] in _BINPREC:
            bp = _BINPREC[self.cur[0]]
            if bp <= prec:
                break
            op = self.next()[0]
            if op == "?":
                bp -= 1                                            # right associative
                t = self.parse_exp()
                self.expect(":")
                f = self.parse_exp(bp)
                left = Expr("sel", op="?", args=[left, t, f])
                continue
            left = Expr("bin", op=op, args=[left, self.parse_exp(bp)])
        return left

    def parse_list(self, fn, begin="(", sep=",", end=")"):
        self.expect(begin)
        out = []
        if self.cur[0] != end:
            while True:
                out.append(fn())
                if not self.accept(sep):
                    break
        self.expect(end)
        return out

    def parse_param(self):
        if self.cur[0] == "ident":
            return Param(self.next()[1], None, [])
        if self.cur[0] not in _SCALAR_TYPES:
            raise TcError(f"expected a scalar type at offset {self.cur[2]}")
        scalar = self.next()[0]
        dims = []
        if self.cur[0] == "(":
            def dim():
                if self.cur[0] == "number":
                    return int(self.parse_const().value)
                return self.expect("ident")[1]
            dims = self.parse_list(dim)
        return Param(self.expect("ident")[1], scalar, dims)

    def parse_where(self):
        look = self.toks[self.p + 1][0]
        if look == "=":
            name = self.expect("ident")[1]
            self.expect("=")
            return ("let", name, self.parse_exp())
        if look == "in":
            name = self.expect("ident")[1]
            self.expect("in")
            lo = self.parse_exp()
            self.expect(":")
            hi = self.parse_exp()
            return ("range", name, lo, hi)
        self.expect("exists")
        return ("exists", self.parse_exp())

    def parse_stmt(self):
        lhs = self.expect("ident")[1]
        idx = []
        if self.cur[0] == "(":
            idx = self.parse_list(lambda: self.expect("ident")[1])
        if self.cur[0] not in _ASSIGN:
            raise TcError(f"expected a valid assignment operator at offset {self.cur[2]}")
        assign = self.next()[0]
        rhs = self.parse_exp()
        if self.accept("<=>"):
            self.expect("ident")
            self.parse_list(self.parse_exp)
        where = []
        if self.accept("where"):
            while True:
                where.append(self.parse_where())
                if not self.accept(","):
                    break
        return Stmt(lhs, idx, assign, rhs, where)

    def parse_def(self):
        self.expect("def")
        name = self.expect("ident")[1]
        params = self.parse_list(self.parse_param)
        self.expect("->")
        rets = self.parse_list(self.parse_param)
        self.expect("{")
        stmts = []
        while not self.accept("}"):
            stmts.append(self.parse_stmt())
        return Def(name, params, rets, stmts)


def parse(src: str) -> Dict[str, Def]:
    """All defs in a TC string, by name (tc/core/compiler.cc:115-124)."""
    p = _Parser(src)
    out = {}
    while p.cur[0] != "eof":
        d = p.parse_def()
        out.setdefault(d.name, d)
    return out


# ----------------------------------------------------------------------------------------------
# Typing (tc/lang/sema.h:129-163) and builtins (tc/lang/builtins.h:23-95)
# ----------------------------------------------------------------------------------------------
BUILTINS = {
    "acos": 1, "acosh": 1, "asin": 1, "asinh": 1, "atan2": 2, "atan": 1, "atanh": 1, "cbrt": 1, "ceil": 1,
    "copysign": 2, "cos": 1, "cosh": 1, "cospi": 1, "cyl_bessel_i0": 1, "cyl_bessel_i1": 1, "erfc": 1,
    "erfcinv": 1, "erfcx": 1, "erf": 1, "erfinv": 1, "exp10": 1, "exp2": 1, "exp": 1, "expm1": 1, "fabs": 1,
    "fdim": 2, "fdivide": 2, "floor": 1, "fma": 3, "fmax": 2, "fmin": 2, "fmod": 2, "hypot": 2, "j0": 1,
    "j1": 1, "lgamma": 1, "log10": 1, "log1p": 1, "log2": 1, "logb": 1, "log": 1, "nextafter": 2,
    "norm3d": 3, "norm4d": 4, "normcdf": 1, "normcdfinv": 1, "pow": 2, "rcbrt": 1, "remainder": 2,
    "rhypot": 2, "rnorm3d": 3, "rnorm4d": 4, "round": 1, "rsqrt": 1, "sin": 1, "sinh": 1, "sinpi": 1,
    "sqrt": 1, "tan": 1, "tanh": 1, "tgamma": 1, "trunc": 1, "y0": 1, "y1": 1,
}


def _canon(t: str) -> str:
    code, bits = _SCALAR_TYPES[t]
    if code == "float":
        return {32: "float", 64: "double", 16: "float16"}[bits]
    if code == "uint":
        return "bool" if bits == 1 else f"uint{bits}"
    return f"int{bits}"


def match_types(a: str, b: str) -> str:
    (ca, ba), (cb, bb) = _SCALAR_TYPES[a], _SCALAR_TYPES[b]
    if (ca, ba) == (cb, bb):
        return _canon(a)
    fa, fb = ca == "float", cb == "float"
    if not fa and fb:
        return _canon(b)
    if fa and not fb:
        return _canon(a)
    if fa and fb:
        return _canon(a if ba > bb else b)
    if ca == "uint" and cb == "uint":
        return _canon(a if ba > bb else b)
    return f"int{max(ba, bb)}"


_CTYPE = {"float16": "_Float16", "float": "float", "double": "double", "int8": "int8_t", "int16": "int16_t", "int32": "int32_t",
          "int64": "int64_t", "uint8": "uint8_t", "uint16": "uint16_t", "uint32": "uint32_t",
          "uint64": "uint64_t", "bool": "uint8_t"}
_NPTYPE = {"float16": np.float16, "float": np.float32, "double": np.float64, "int8": np.int8, "int16": np.int16, "int32": np.int32,
           "int64": np.int64, "uint8": np.uint8, "uint16": np.uint16, "uint32": np.uint32,
           "uint64": np.uint64, "bool": np.uint8}


# ----------------------------------------------------------------------------------------------
# Semantic analysis + range inference on concrete sizes
# ----------------------------------------------------------------------------------------------
@dataclass
class Tensor:
    name: str
    scalar: str
    mins: List[int]
    extents: List[int]
    arg_names: List[str] = field(default_factory=list)   # index names of the first definition


class Analysis:
    """A Def specialised on concrete input shapes: typed statements with index ranges."""

    def __init__(self, d: Def, input_shapes: Sequence[Sequence[int]]):
        self.d = d
        self.warnings: List[str] = []
        self.sizes: Dict[str, int] = {}
        self.tensors: Dict[str, Tensor] = {}
        self.inputs: List[str] = []
        if len(input_shapes) != len(d.params):
            raise TcError(f"expected {len(d.params)} inputs but got {len(input_shapes)}")
        for p, shape in zip(d.params, input_shapes):
            if p.scalar is None:
                raise TcError(f"input {p.name} needs a type")
            if len(shape) != len(p.dims):
                raise TcError(f"expected a tensor with {len(p.dims)} dimensions but found {len(shape)} dimensions.")
            for dim, s in zip(p.dims, shape):      # halide_utils.cc:41-86
                if isinstance(dim, int):
                    if dim != s:
                        raise TcError(f"Constant dimension expected size {dim} but found {s}")
                elif dim in self.sizes:
                    if self.sizes[dim] != s:
                        raise TcError(f"Mismatched sizes for dimension {dim} previous value is {self.sizes[dim]} but found {s} here")
                else:
                    self.sizes[dim] = int(s)
            if p.name in self.tensors or p.name in BUILTINS:
                raise TcError(f"{p.name} already defined")
            self.tensors[p.name] = Tensor(p.name, _canon(p.scalar), [0] * len(shape), [int(s) for s in shape])
            self.inputs.append(p.name)
        self.outputs = [r.name for r in d.returns]
        self._written: set = set()
        self._bounds_by_name: Dict[str, Dict[str, Tuple[int, int]]] = {}
        self.annotated = {r.name: r for r in d.returns if r.scalar is not None}
        for s in d.stmts:
            self._check_stmt(s)
        for o in self.outputs:
            if o not in self.tensors:
                raise TcError(f"undefined variable {o} used here.")
        # a tensor has one bound, that of its last definition, applied to all its stages
        # (tc2halide.cc:676-693, :808-870): an earlier statement inferred over a larger range
        # writes only inside it
        for s in d.stmts:
            t = self.tensors[s.lhs]
            for dim, v in enumerate(s.indices):
                lo, hi = s.ranges[v]
                lo, hi = max(lo, t.mins[dim]), min(hi, t.mins[dim] + t.extents[dim] - 1)
                s.ranges[v] = (lo, hi)

    # -- typing ---------------------------------------------------------------------------
    def _type(self, e: Expr, s: Stmt, index_env: Dict[str, None], lets: Dict[str, Expr], allow_access=True) -> Expr:
        k = e.kind
        if k == "const":
            return e
        if k == "ident":
            if e.op in index_env:
                e.type = "int32"
                return e
            if e.op in lets:
                return lets[e.op]
            if e.op in self.sizes:
                e.type = "int32"
                e.kind = "size"
                return e
            if e.op in self.tensors:
                if len(self.tensors[e.op].extents) != 0:
                    raise TcError("expected a scalar but found a tensor expression.")
                return self._type(Expr("apply", op=e.op, args=[]), s, index_env, lets, allow_access)
            # unknown identifier -> reduction variable (sema.h:230-240)
            index_env[e.op] = None
            s.reduction_vars.append(e.op)
            e.type = "int32"
            return e
        if k == "apply":
            if not allow_access:
                raise TcError("tensor accesses cannot be used in this context")
            if e.op in BUILTINS:
                if BUILTINS[e.op] != len(e.args):
                    raise TcError(f"expected {BUILTINS[e.op]} but found {len(e.args)}")
                args = [self._type(a, s, index_env, lets) for a in e.args]
                ty = "float"
                for a in args:
                    ty = match_types(ty, a.type)
                return Expr("builtin", op=e.op, args=args, type=ty)
            if e.op not in self.tensors:
                raise TcError(f"undefined variable {e.op} used here.")
            t = self.tensors[e.op]
            if len(t.extents) != len(e.args):
                raise TcError(f"expected {len(t.extents)} dimensions but found {len(e.args)} dimensions.")
            args = [self._type(a, s, index_env, lets) for a in e.args]
            for a in args:
                if _SCALAR_TYPES[a.type][0] == "float":
                    raise TcError(f" expected integral type but found {a.type}")
            return Expr("access", op=e.op, args=args, type=t.scalar)
        if k == "bin":
            args = [self._type(a, s, index_env, lets, allow_access) for a in e.args]
            mt = match_types(args[0].type, args[1].type)
            if e.op in ("+", "-", "*", "/", "%", "min", "max"):
                ty = mt
            elif e.op in ("==", "!=", ">=", "<=", "<", ">"):
                ty = "bool"
            else:                                                   # && ||
                if mt != "bool":
                    raise TcError(f"expected boolean but found {mt}")
                ty = "bool"
            return Expr("bin", op=e.op, args=args, type=ty)
        if k == "un":
            a = self._type(e.args[0], s, index_env, lets, allow_access)
            if e.op == "!":
                if a.type != "bool":
                    raise TcError(f"expected boolean but found {a.type}")
                return Expr("un", op="!", args=[a], type="bool")
            return Expr("un", op="-", args=[a], type=a.type)
        if k == "sel":
            c, t, f = [self._type(a, s, index_env, lets, allow_access) for a in e.args]
            if c.type != "bool":
                raise TcError(f"expected boolean but found {c.type}")
            return Expr("sel", op="?", args=[c, t, f], type=match_types(t.type, f.type))
        if k == "cast":
            a = self._type(e.args[0], s, index_env, lets, allow_access)
            return Expr("cast", op=_canon(e.op), args=[a], type=_canon(e.op))
        raise TcError(f"NYI - semantic checking for {k}")

    # -- affine view of a subscript ---------------------------------------------------------
    def _affine(self, e: Expr) -> Optional[Dict[str, int]]:
        """{var: coef, '': const} or None when the expression is not integer-affine."""
        k = e.kind
        if k == "const":
            return {"": int(e.value)} if e.type == "int32" else None
        if k == "size":
            return {"": self.sizes[e.op]}
        if k == "ident":
            return {e.op: 1, "": 0}
        if k == "un" and e.op == "-":
            a = self._affine(e.args[0])
            return None if a is None else {v: -c for v, c in a.items()}
        if k == "bin" and e.op in ("+", "-"):
            a, b = self._affine(e.args[0]), self._affine(e.args[1])
            if a is None or b is None:
                return None
            out = dict(a)
            sg = 1 if e.op == "+" else -1
            for v, c in b.items():
                out[v] = out.get(v, 0) + sg * c
            return out
        if k == "bin" and e.op == "*":
            a, b = self._affine(e.args[0]), self._affine(e.args[1])
            if a is None or b is None:
                return None
            ca = len([v for v in a if v and a[v]]) == 0
            cb = len([v for v in b if v and b[v]]) == 0
            if ca:
                return {v: a.get("", 0) * c for v, c in b.items()} | ({"": a.get("", 0) * b.get("", 0)})
            if cb:
                return {v: b.get("", 0) * c for v, c in a.items()} | ({"": a.get("", 0) * b.get("", 0)})
            return None
        return None

    def _vars_of(self, e: Expr, out: List[str]):
        if e.kind == "ident":
            if e.op not in out:
                out.append(e.op)
        for a in e.args:
            self._vars_of(a, out)

    def _collect(self, e: Expr, cons: List[tuple], free: List[str]):
        """Walk the RHS: free variables and 'access in bounds' constraints (tc2halide.cc:276-330)."""
        if e.kind == "ident" and e.op not in free:
            free.append(e.op)
        for a in e.args:
            self._collect(a, cons, free)
        if e.kind == "access":
            t = self.tensors[e.op]
            for d, a in enumerate(e.args):
                lo, hi = t.mins[d], t.mins[d] + t.extents[d] - 1
                aff = self._affine(a)
                if aff is None:
                    vs: List[str] = []
                    self._vars_of(a, vs)
                    cons.append(("opaque", vs))
                else:
                    c0 = aff.get("", 0)
                    coefs = {v: c for v, c in aff.items() if v and c}
                    cons.append(("ge", dict(coefs), c0 - lo))                       # expr - lo >= 0
                    cons.append(("ge", {v: -c for v, c in coefs.items()}, hi - c0))  # hi - expr >= 0

    def _const_int(self, e: Expr) -> int:
        a = self._affine(e)
        if a is None or any(v for v in a if v and a[v]):
            raise TcError("range bounds must be integer expressions of the sizes")
        return a.get("", 0)

    # -- one statement ---------------------------------------------------------------------
    def _check_stmt(self, s: Stmt):
        if s.lhs in self.inputs:
            raise TcError("TC inputs are immutable")
        index_env: Dict[str, None] = {}
        for i in s.indices:
            if i in index_env or i in BUILTINS:
                raise TcError(f"{i} already defined")
            index_env[i] = None
        lets: Dict[str, Expr] = {}
        s.reduction_vars = []
        solution: Dict[str, Tuple[int, int]] = {}
        exists: List[Expr] = []
        for w in s.where:
            if w[0] == "let":
                lets[w[1]] = self._type(w[2], s, index_env, lets)
            elif w[0] == "range":
                if w[1] not in index_env:
                    index_env[w[1]] = None
                    s.reduction_vars.append(w[1])
                lo = self._type(w[2], s, index_env, lets, allow_access=False)
                hi = self._type(w[3], s, index_env, lets, allow_access=False)
                solution[w[1]] = (self._const_int(lo), self._const_int(hi) - 1)   # tc2halide.cc:652-669
            else:
                exists.append(self._type(w[1], s, index_env, lets))
        s.rhs = self._type(s.rhs, s, index_env, lets)
        scalar = s.rhs.type
        if s.lhs in self.annotated:
            ann = self.annotated[s.lhs]
            if _canon(ann.scalar) != match_types(scalar, ann.scalar):
                raise TcError(f" attempting to assign type {scalar} to narrower type {ann.scalar} without an explicit cast")
            if len(ann.dims) != len(s.indices):
                raise TcError(f" tensor defined with {len(s.indices)} dimensions but declared as an output with {len(ann.dims)} dimensions.")
            scalar = _canon(ann.scalar)
        if s.lhs in self.tensors and s.lhs not in self.inputs:
            # a later statement keeps the type of the tensor's first definition; Halide refuses an
            # update definition of another type (tc2halide.cc builds one Func per tensor), so a
            # value that would lose precision is an error as it is for annotated outputs
            have = self.tensors[s.lhs].scalar
            if _canon(have) != match_types(scalar, have):
                raise TcError(f" attempting to assign type {scalar} to narrower type {have} without an explicit cast")
            # ... and an update definition with another number of arguments (the reference's sema
            # lets it through, tc/lang/sema.h:566-571)
            if len(self.tensors[s.lhs].extents) != len(s.indices):
                raise TcError(f"{s.lhs} was defined with {len(self.tensors[s.lhs].extents)} dimensions and is written here with {len(s.indices)}")
        if s.assign in ("+=", "*=", "min=", "max=") and s.lhs not in self.tensors:
            self.warnings.append(f"Reduction without initialization. If {s.lhs} is not pre-initialized ...")
        if s.lhs not in self.outputs:
            raise TcError(f"{s.lhs} is not listed as an input or output to this function. Temporaries tensors are not yet implemented")
        if not s.reduction_vars and s.assign.endswith("!"):
            s.assign = "="                                           # sema.h:588-590
        if s.reduction_vars and s.assign == "=":
            raise TcError(f"this statement includes reduction variable '{s.reduction_vars[-1]}' but does not specify a reduction.")
        s.scalar = scalar

        # ---- forward range inference (tc2halide.cc:270-498), on concrete sizes -----------------
        cons: List[tuple] = []
        free: List[str] = []
        for ex in exists:
            self._collect(ex, cons, free)
        self._collect(s.rhs, cons, free)
        unsolved = sorted(v for v in free if v not in solution)

        def eliminate(c):
            """Worst case of a 'coefs.x + k >= 0' inequality over the solved variables."""
            if c[0] == "opaque":
                vs = [v for v in c[1] if v not in solution]
                return ("opaque", vs) if vs else ("dropped",)
            coefs, k0 = dict(c[1]), c[2]
            for v in list(coefs):
                if v in solution:
                    lo, hi = solution[v]
                    k0 += coefs[v] * (lo if coefs[v] > 0 else hi)
                    del coefs[v]
            return ("ge", coefs, k0)

        def settle(cs, had_vars):
            out = []
            for c, hv in zip(cs, had_vars):
                if c[0] == "dropped":
                    self.warnings.append("Required precondition will not be checked at runtime (non-affine subscript)")
                elif c[0] == "ge" and not c[1]:
                    if c[2] < 0 and hv:
                        self.warnings.append("Required precondition will not be checked at runtime")
                    elif c[2] < 0:
                        self.warnings.append("Required precondition will not be checked at runtime")
                else:
                    out.append(c)
            return out

        hv = [bool(c[1]) for c in cons]
        cons = settle([eliminate(c) for c in cons], hv)
        while unsolved:
            still = []
            for v in unsolved:
                mine, rest = [], []
                for c in cons:
                    if c[0] == "ge" and set(c[1]) == {v}:
                        mine.append(c)
                    else:
                        rest.append(c)
                lo, hi = -math.inf, math.inf
                for _, coefs, k0 in mine:
                    a = coefs[v]
                    if a > 0:                       # a v + k0 >= 0  ->  v >= ceil(-k0/a)
                        lo = max(lo, -(k0 // a))
                    else:                           # v <= floor(k0/(-a))
                        hi = min(hi, k0 // (-a))
                if lo != -math.inf and hi != math.inf and lo > hi:
                    raise TcError(f"Inferred an empty range for variable {v}.")
                if lo == -math.inf or hi == math.inf:
                    still.append(v)
                else:
                    solution[v] = (int(lo), int(hi))
                    cons = rest
            hv = [bool(c[1]) for c in cons]
            cons = settle([eliminate(c) for c in cons], hv)
            if len(still) == len(unsolved):
                raise TcError("Could not infer ranges for free variables. Use a where clause: " + ", ".join(unsolved))
            unsolved = still
        for v in s.indices:
            if v not in solution:
                raise TcError(f"Free variable {v} was not solved in range inference. May not be used right-hand side")
        # reduction variables = RHS variables not on the LHS, first appearance order (tc2halide.cc:698-740)
        order: List[str] = []
        self._vars_of(s.rhs, order)
        s.reduction_vars = [v for v in order if v not in s.indices]
        for v in s.reduction_vars:
            if v not in solution:
                raise TcError(f"Free variable {v} is unconstrained. Use a 'where' clause to set its range.")
        s.ranges = {v: solution[v] for v in list(s.indices) + s.reduction_vars}

        # record / clobber the LHS tensor's bounds (tc2halide.cc:689-693)
        if s.lhs not in self.tensors:
            self.tensors[s.lhs] = Tensor(s.lhs, scalar, [0] * len(s.indices), [0] * len(s.indices), list(s.indices))
            self._bounds_by_name[s.lhs] = {}
        t = self.tensors[s.lhs]
        by_name = self._bounds_by_name[s.lhs]
        for v in s.indices:
            by_name[v] = solution[v]
        for d, a in enumerate(t.arg_names):
            lo, hi = by_name[a]
            t.mins[d], t.extents[d] = lo, hi - lo + 1
        self._written.add(s.lhs)

    # -- results ---------------------------------------------------------------------------
    def output_shapes(self) -> List[Tuple[str, str, List[int]]]:
        return [(o, self.tensors[o].scalar, list(self.tensors[o].extents)) for o in self.outputs]


def analyze(tc: str, entry: str, input_shapes) -> Analysis:
    defs = parse(tc)
    if entry not in defs:
        raise TcError(f"attempting to access undefined function {entry}")
    return Analysis(defs[entry], input_shapes)


def infer_output_shapes(tc: str, entry: str, input_shapes):
    return analyze(tc, entry, input_shapes).output_shapes()


# ----------------------------------------------------------------------------------------------
# C emission of the canonical loop nest
# ----------------------------------------------------------------------------------------------
_IDENT = {"+": "0", "*": "1"}


def _identity(op: str, scalar: str) -> str:
    """Reduction identities (tc2halide.cc:574-601): 0, 1, type max, type min."""
    base = op.rstrip("!").rstrip("=")
    if scalar == "float16":                         # the largest finite half is 65504
        return {"+": "((_Float16)0.0f)", "*": "((_Float16)1.0f)", "min": "((_Float16)65504.0f)",
                "max": "((_Float16)-65504.0f)"}[base]
    fl = scalar in ("float", "double")
    if base == "+":
        return "0.000000f" if scalar == "float" else ("0.0" if fl else "0")
    if base == "*":
        return "1.000000f" if scalar == "float" else ("1.0" if fl else "1")
    info = np.finfo(_NPTYPE[scalar]) if fl else np.iinfo(_NPTYPE[scalar])
    v = info.max if base == "min" else info.min
    if scalar == "float":
        return f"{float(v)!r}f".replace("e+", "e")
    if fl:
        return repr(float(v))
    if scalar == "uint64":
        return f"{int(v)}ULL"
    if scalar == "int64":
        return f"({int(v) + 1}LL - 1)" if v < 0 else f"{int(v)}LL"   # (-2^63 has no literal of its own)
    return str(int(v))


class _CEmitter:
    def __init__(self, an: Analysis):
        self.an = an

    def index(self, name: str, args: List[str]) -> str:
        t = self.an.tensors[name]
        if not args:
            return f"{name}[0]"
        # storage starts at the inferred lower bound: element k of a dimension holds point min + k
        # (a Halide buffer whose min is set, tc2halide.cc:903, is addressed this way by the CPU JIT)
        rel = [a if t.mins[d] == 0 else f"({a} - {t.mins[d]})" for d, a in enumerate(args)]
        flat = rel[0]
        if int(np.prod([int(e) for e in t.extents], dtype=np.int64)) >= 2 ** 31:
            flat = f"(int64_t)({flat})"                 # element offsets beyond 32 bits
        for d in range(1, len(args)):
            flat = f"({flat})*{t.extents[d]} + ({rel[d]})"
        return f"{name}[{flat}]"

    def pretty_index(self, name, args):
        return name + "".join(f"[{a}]" for a in args)

    def expr(self, e: Expr, rename, pretty=False) -> str:
        k = e.kind
        if k == "const":
            if e.type == "float":
                return f"{e.value:.6f}f" if pretty else f"{np.float32(e.value).item()!r}f"
            return str(int(e.value))
        if k == "size":
            return e.op if pretty else str(self.an.sizes[e.op])
        if k == "ident":
            return rename(e.op)
        if k == "access":
            args = [self.expr(a, rename, pretty) for a in e.args]
            return self.pretty_index(e.op, args) if pretty else self.index(e.op, args)
        if k == "builtin":
            if e.type == "float16" and not pretty:   # no half math library: evaluated in float, rounded once
                return f"((_Float16){e.op}f(" + ", ".join(self.cast(a, "float", rename) for a in e.args) + "))"
            fn = e.op + ("f" if e.type == "float" and not pretty else "")
            return f"{fn}(" + ", ".join(self.cast(a, e.type, rename, pretty) for a in e.args) + ")"
        if k == "cast":
            return f"(({_CTYPE[e.op]})({self.expr(e.args[0], rename, pretty)}))"
        if k == "un":
            if e.op == "-":
                zero = "0.000000f" if (pretty and e.type == "float") else ("0.0f" if e.type == "float" else "0")
                return f"({zero} - {self.expr(e.args[0], rename, pretty)})"
            return f"(!{self.expr(e.args[0], rename, pretty)})"
        if k == "sel":
            c, t, f = e.args
            return f"({self.expr(c, rename, pretty)} ? {self.cast(t, e.type, rename, pretty)} : {self.cast(f, e.type, rename, pretty)})"
        if k == "bin":
            a, b = e.args
            mt = match_types(a.type, b.type)
            sa, sb = self.cast(a, mt, rename, pretty), self.cast(b, mt, rename, pretty)
            if e.op in ("min", "max"):
                if pretty:
                    return f"{e.op}({sa}, {sb})"
                if mt == "float16":
                    return f"((_Float16)f{e.op}f((float)({sa}), (float)({sb})))"
                if mt in ("float", "double"):
                    return f"{'fminf' if e.op == 'min' else 'fmaxf'}({sa}, {sb})" if mt == "float" else f"f{e.op}({sa}, {sb})"
                return f"(({sa}) {'<' if e.op == 'min' else '>'} ({sb}) ? ({sa}) : ({sb}))"
            if e.op == "%" and mt == "float16" and not pretty:
                return f"((_Float16)fmodf((float)({sa}), (float)({sb})))"
            if e.op in ("/", "%") and mt not in ("float16", "float", "double") and not pretty:
                if mt.startswith("uint") or mt == "bool":
                    return f"({sa} {e.op} {sb})"     # unsigned: rounding down is truncation (and 2^63.. must not pass through int64)
                return f"tc_floor{'div' if e.op == '/' else 'mod'}({sa}, {sb})"   # Halide integer semantics
            if e.op == "%" and mt in ("float", "double") and not pretty:
                return f"fmod{'f' if mt == 'float' else ''}({sa}, {sb})"
            if pretty and e.op in ("*", "/", "%"):
                return f"({sa}{e.op}{sb})"
            return f"({sa} {e.op} {sb})"
        raise TcError(f"cannot emit {k}")

    def cast(self, e: Expr, to: str, rename, pretty=False) -> str:
        s = self.expr(e, rename, pretty)
        if pretty or e.type == to or to == "bool":
            return s
        return f"(({_CTYPE[to]})({s}))"

    def stmt_nests(self, s: Stmt, pretty=False) -> List[str]:
        """One or two loop nests for a statement (init nest for 'op=!', then the update nest)."""
        an = self.an
        lines: List[str] = []
        t = an.tensors[s.lhs]
        stage = getattr(self, "_stage", {})
        self._stage = stage

        def nest(loop_vars, body_fn):
            st = stage.get(s.lhs, 0)
            stage[s.lhs] = st + 1
            ren = (lambda v: f"{s.lhs}_s{st}_{v}") if True else None
            ind = ""
            for v in loop_vars:
                lo, hi = s.ranges[v]
                ub = self._pretty_bounds.get((s.lhs, v), str(hi + 1)) if pretty else str(hi + 1)
                lines.append(f"{ind}for (int {ren(v)} = {lo}; {ren(v)} < {ub}; {ren(v)}++) {{")
                ind += "  "
            lines.append(ind + body_fn(ren))
            for _ in loop_vars:
                ind = ind[:-2]
                lines.append(ind + "}")

        def lhs_ref(ren):
            args = [ren(v) for v in s.indices]
            return self.pretty_index(s.lhs, args) if pretty else self.index(s.lhs, args)

        base = s.assign.rstrip("!")
        if s.assign.endswith("!"):
            nest(list(s.indices), lambda ren: f"{lhs_ref(ren)} = {_identity(s.assign, s.scalar)};")
        loops = list(s.indices) + list(s.reduction_vars)

        def body(ren):
            rhs = self.cast(s.rhs, s.scalar, ren, pretty)
            l = lhs_ref(ren)
            if base == "=":
                return f"{l} = {rhs};"
            if base == "+=":
                return f"{l} = ({l} + {rhs});"
            if base == "*=":
                return f"{l} = ({l}*{rhs});" if pretty else f"{l} = ({l} * {rhs});"
            fn = "min" if base == "min=" else "max"
            if pretty:
                return f"{l} = {fn}({l}, {rhs});"
            if s.scalar == "float16":
                return f"{l} = (_Float16)f{fn}f((float)({l}), (float)({rhs}));"
            if s.scalar in ("float", "double"):
                f = ("fminf" if fn == "min" else "fmaxf") if s.scalar == "float" else "f" + fn
                return f"{l} = {f}({l}, {rhs});"
            return f"{l} = (({l}) {'<' if fn == 'min' else '>'} ({rhs}) ? ({l}) : ({rhs}));"
        nest(loops, body)
        return lines

    _pretty_bounds: Dict[Tuple[str, str], str] = {}


def emit_loop_nest_text(an: Analysis, symbolic_bounds: Optional[Dict[Tuple[str, str], str]] = None) -> str:
    """The nest in the spelling of the reference's Halide C printout (test/test_core.cc:93-232):
    N-d subscripts, `<tensor>_s<stage>_<var>` loop names.  `symbolic_bounds[(tensor, var)]`
    optionally replaces a numeric upper bound by the caller's text."""
    em = _CEmitter(an)
    em._pretty_bounds = symbolic_bounds or {}
    out: List[str] = []
    for s in an.d.stmts:
        out += em.stmt_nests(s, pretty=True)
    return "\n".join(out) + "\n"


_PRELUDE = """#include <stdint.h>
#include <math.h>
static inline int64_t tc_floordiv(int64_t a, int64_t b) { int64_t q = a / b; return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q; }
static inline int64_t tc_floormod(int64_t a, int64_t b) { return a - tc_floordiv(a, b) * b; }
/* device builtins libm lacks (tc/lang/builtins.h:23-95 names them after the CUDA math library) */
static inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
static inline double rsqrt(double x) { return 1.0 / sqrt(x); }
"""


def emit_c(an: Analysis, fname: str = "tc_oracle_kernel") -> str:
    """C source: void f(const T* in..., T* out...) — inputs then outputs, as the CPU JIT orders
    them (codegen_llvm.cc:343-387); sizes are baked in as constants."""
    em = _CEmitter(an)
    sig = []
    for i in an.inputs:
        sig.append(f"const {_CTYPE[an.tensors[i].scalar]}* __restrict__ {i}")
    for o in an.outputs:
        sig.append(f"{_CTYPE[an.tensors[o].scalar]}* __restrict__ {o}")
    body: List[str] = []
    for s in an.d.stmts:
        body += ["  " + l for l in em.stmt_nests(s)]
    return _PRELUDE + f"void {fname}(" + ", ".join(sig) + ") {\n" + "\n".join(body) + "\n}\n"


# ----------------------------------------------------------------------------------------------
# Build + run
# ----------------------------------------------------------------------------------------------
_BUILD_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_build")
_CLANG = os.environ.get("TC_ORACLE_CLANG", "/opt/rocm/llvm/bin/clang")
_CFLAGS = ["-O3", "-ffp-contract=off", "-fno-fast-math", "-shared", "-fPIC"]
_cache: Dict[str, ctypes.CDLL] = {}


def build(an: Analysis, native: bool = False, in_tree: bool = False) -> ctypes.CDLL:
    """Compile the nest.  The library goes to a per-host temporary directory (hundreds of test
    nests do not belong next to the sources, and one built with `native=True`, i.e. -march=native,
    must not travel to another machine); `in_tree=True` keeps it under oracle/_build instead (the
    build check of the benchmark configurations)."""
    src = emit_c(an)
    flags = _CFLAGS + (["-march=native"] if native else [])
    key = hashlib.sha1((src + " ".join(flags)).encode()).hexdigest()[:16]
    if key in _cache:
        return _cache[key]
    tmp_root = os.environ.get("TC_ORACLE_BUILD_DIR") or os.path.join(tempfile.gettempdir(), f"tc_oracle_{os.getuid()}")
    bdir = _BUILD_DIR if in_tree else os.path.join(tmp_root, "native" if native else "portable")
    os.makedirs(bdir, exist_ok=True)
    so = os.path.join(bdir, f"oracle_{an.d.name}_{key}.so")
    if not os.path.exists(so):
        c = os.path.join(bdir, f"oracle_{an.d.name}_{key}.c")
        with open(c, "w") as f:
            f.write(src)
        tmp = so + f".tmp{os.getpid()}"
        # gcc 11 has no _Float16 on x86-64: nests with half tensors go through the ROCm clang, every
        # operation rounded to half (no excess precision carried from one operation to the next)
        half = any(t.scalar == "float16" for t in an.tensors.values())
        cc = [_CLANG, "-fexcess-precision=16"] if half else ["gcc"]
        subprocess.run([*cc, *flags, "-o", tmp, c, "-lm"], check=True)
        os.replace(tmp, so)
    lib = ctypes.CDLL(so)
    _cache[key] = lib
    return lib


def refuse_empty_ranges(an: "Analysis"):
    """Range inference accepts `where i in 8:4` and reports a negative extent, as the reference's
    does (test/test_inference.cc:498-511, "silently infers a negative size"); nothing can be run
    over such a range, so executing the definition is refused."""
    for s in an.d.stmts:
        for v, (lo, hi) in s.ranges.items():
            if hi < lo:
                raise TcError(f"Empty range for variable {v}: {lo}:{hi + 1}.")


def run(tc: str, entry: str, inputs: Sequence[np.ndarray], outputs: Optional[Sequence[np.ndarray]] = None,
        native: bool = False):
    """Execute `entry` on numpy inputs with the compiled canonical loop nest.  Returns the list
    of output arrays.  `outputs` may carry pre-existing values for non-initialising reductions."""
    an = analyze(tc, entry, [a.shape for a in inputs])
    refuse_empty_ranges(an)
    for name, a in zip(an.inputs, inputs):
        want = _NPTYPE[an.tensors[name].scalar]
        if an.tensors[name].scalar == "bool" and a.dtype == np.bool_:
            continue                                   # numpy's own bool: one byte holding 0 or 1, as the kernel reads it
        if a.dtype != want:
            raise TcError(f"expected type {an.tensors[name].scalar} but found {a.dtype}")
    lib = build(an, native)
    ins = [np.ascontiguousarray(a) for a in inputs]
    if outputs is None:
        outs = [np.zeros(shape, dtype=_NPTYPE[sc]) for _, sc, shape in an.output_shapes()]
    else:
        outs = [np.ascontiguousarray(o) for o in outputs]
    fn = lib.tc_oracle_kernel
    fn.restype = None
    fn(*[ctypes.c_void_p(a.ctypes.data) for a in ins + outs])
    return outs


def run_python(tc: str, entry: str, inputs: Sequence[np.ndarray], acc_dtype=None):
    """Pure-Python execution of the same nest for tiny shapes (float32 arithmetic per operation
    unless acc_dtype is given, e.g. np.float64 for a brute-force high-precision answer)."""
    an = analyze(tc, entry, [a.shape for a in inputs])
    refuse_empty_ranges(an)
    env = {n: np.asarray(a) for n, a in zip(an.inputs, inputs)}
    for o, sc, shape in an.output_shapes():
        env[o] = np.zeros(shape, dtype=acc_dtype or _NPTYPE[sc])

    def ev(e: Expr, idx):
        k = e.kind
        if k == "const":
            return (acc_dtype or np.float32)(e.value) if e.type == "float" else int(e.value)
        if k == "size":
            return an.sizes[e.op]
        if k == "ident":
            return idx[e.op]
        if k == "access":
            v = env[e.op][tuple(int(ev(a, idx)) - m for a, m in zip(e.args, an.tensors[e.op].mins))]
            return acc_dtype(v) if acc_dtype and e.type in ("float16", "float", "double") else v
        if k == "bin":
            a, b = ev(e.args[0], idx), ev(e.args[1], idx)
            mt = match_types(e.args[0].type, e.args[1].type)
            if mt in ("float16", "float", "double"):
                ty = acc_dtype or _NPTYPE[mt]
                a, b = ty(a), ty(b)
            op = e.op
            if op == "+": return a + b
            if op == "-": return a - b
            if op == "*": return a * b
            if op == "/": return a / b if mt in ("float16", "float", "double") else a // b
            if op == "%": return math.fmod(a, b) if mt in ("float16", "float", "double") else a % b
            if op == "min": return min(a, b)
            if op == "max": return max(a, b)
            return {"==": a == b, "!=": a != b, "<": a < b, ">": a > b, "<=": a <= b, ">=": a >= b,
                    "&&": bool(a) and bool(b), "||": bool(a) or bool(b)}[op]
        if k == "un":
            v = ev(e.args[0], idx)
            return -v if e.op == "-" else (not v)
        if k == "sel":
            return ev(e.args[1], idx) if ev(e.args[0], idx) else ev(e.args[2], idx)
        if k == "cast":
            return _NPTYPE[e.op](ev(e.args[0], idx))
        if k == "builtin":
            fn = getattr(np, {"fabs": "abs"}.get(e.op, e.op))
            return (acc_dtype or np.float32)(fn(*[np.float64(ev(a, idx)) for a in e.args]))
        raise TcError(k)

    import itertools
    for s in an.d.stmts:
        out = env[s.lhs]
        base = s.assign.rstrip("!")
        lhs_ranges = [range(s.ranges[v][0], s.ranges[v][1] + 1) for v in s.indices]
        lo = tuple(an.tensors[s.lhs].mins)               # storage starts at the inferred lower bound
        red_ranges = [range(s.ranges[v][0], s.ranges[v][1] + 1) for v in s.reduction_vars]
        if s.assign.endswith("!"):
            ident = {"+=": 0, "*=": 1, "min=": np.inf, "max=": -np.inf}[base]
            for q in itertools.product(*lhs_ranges):
                out[tuple(a - b for a, b in zip(q, lo))] = ident
        for q in itertools.product(*lhs_ranges):
            idx = dict(zip(s.indices, q))
            p = tuple(a - b for a, b in zip(q, lo))
            for r in itertools.product(*red_ranges):
                idx.update(zip(s.reduction_vars, r))
                v = ev(s.rhs, idx)
                if base == "=": out[p] = v
                elif base == "+=": out[p] = out[p] + v
                elif base == "*=": out[p] = out[p] * v
                elif base == "min=": out[p] = min(out[p], v)
                else: out[p] = max(out[p], v)
    return [env[o] for o in an.outputs]
