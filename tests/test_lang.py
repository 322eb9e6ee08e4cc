"""Front end (lexer, parser, semantic analysis) of the C++ library against the reference's golden
dumps (fixtures under tests/golden/lang, produced by tests/golden/make_lang_fixtures.py) and the
error / warning known answers of test/test_lang.cc:270-370 and test/cuda/test_corner_cases.cc."""
import os

import pytest

import tensorcomprehensions_amd as tc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lang")


def golden(name):
    return open(os.path.join(GOLDEN, name)).read()


CONV = """
    def conv(float(B,IP,H,W) input, float(OP,IP,KH,KW) weight) -> (output) {
      output(b, op, h, w) +=! input(b, ip, h + kh, w + kw) * weight(op, ip, kh, kw)
    }
  """


def test_lexer_tokens_and_highlight():
    text = "min min+max 1.4 .3 3 3.\n3e-3 .5e-7 3E-5 foobar"
    assert tc.lang_dump(text, "lexer") == golden("lexer.expected")


@pytest.mark.parametrize("text,what,fixture", [
    ("-3%2+4*5+7-a", "exp", "math.expected"),
    ("foo(3,4,5+6,a)", "exp", "function.expected"),
    ("a ? 3 : b ? 3 : 4", "exp", "trinary.expected"),
    ("R(i,j) +=! A(i,j) * B(j,k)", "stmt", "comprehension.expected"),
    ("output(b, op, h, w) +=! input(b, ip, h + kh, w + kw) * weight(op, ip, kh, kw)", "stmt", "statement.expected"),
    (CONV, "function", "convolution.expected"),
    ("""
    def fun(float(M) I) -> (O) {
      O +=! I(i)
    }
  """, "function", "scalar.expected"),
    (CONV, "sema", "sema.expected"),
    (CONV, "sema_env", "sema-env.expected"),
    ("""
    def fun(float(M) I) -> (O) {
      O +=! log(tanh(I(i)))
    }
  """, "sema+env", "builtins.expected"),
    ("""
    def fun(float(M) A, float(N) B) -> (O) {
      O +=! A(int32(B(i)))
    }
  """, "sema+env", "indirect.expected"),
    ("""
    def fun(float(M) A, float(N) B) -> (O) {
      O max=! A(int32(B(i)))
    }
  """, "sema+env", "maxeq.expected"),
    ("""
    def fun(float(X,Y) A, float(Y,Z) B) -> (O) {
      O(i,j) +=! A(i,k) * B(k,j) <=> matmul(A(i,k), B(k,j))
    }
  """, "sema+env", "annotate.expected"),
])
def test_dump_matches_golden(text, what, fixture):
    assert tc.lang_dump(text, what) == golden(fixture)


def test_left_associativity():
    d = tc.lang_dump("a + b + c", "exp")
    assert d.replace("\n", " ").split() == "(+ (+ (ident a) (ident b)) (ident c))".split()


def test_comments_are_skipped():
    text = """#beginning comment
    def fun(float(M) A, float(N) B) -> (O) {
      # two lines of comments
      # in a row, also a keyword def ->
      O max=! A(int32(B(i)))
    }
  #terminal comment"""
    assert "max_eq_b" in tc.lang_dump(text, "sema")


@pytest.mark.parametrize("fragment,text", [
    ("but does not specify a reduction", "def fun(float(M,N) A) -> (O) { O(i) = A(i,j) }"),
    ("TC inputs are immutable", "def fun(float(M) A) -> (O) { A(i) = A(i) \n O(i) = A(i) }"),
    ("Temporaries tensors are not yet implemented", "def fun(float(M) A) -> (O) { T(i) = A(i) \n O(i) = T(i) }"),
    ("expected 2 dimensions but found 1 dimensions", "def fun(float(M,N) A) -> (O) { O(i) = A(i) }"),
    ("expected integral type", "def fun(float(M) A, float(M) B) -> (O) { O(i) = A(B(i)) }"),
    ("tensor accesses cannot be used in this context", "def fun(float(M) A) -> (O) { O(i) = A(i) where i in 0:A(0) }"),
    ("is a built-in function and cannot be redefined", "def fun(float(M) exp) -> (O) { O(i) = exp(i) }"),
    ("already defined", "def fun(float(M) A, float(M) A) -> (O) { O(i) = A(i) }"),
    ("undefined variable", "def fun(float(M) A) -> (O) { O(i) = Q(i) }"),
    ("expected boolean", "def fun(float(M) A) -> (O) { O(i) = A(i) ? 1.0 : 2.0 }"),
    ("without an explicit cast", "def fun(float(M) A) -> (int32(M) O) { O(i) = A(i) }"),
    ("expected (", "def fun float(M) A) -> (O) { O(i) = A(i) }"),
    ("a valid assignment operator", "def fun(float(M) A) -> (O) { O(i) A(i) }"),
])
def test_front_end_errors(fragment, text):
    with pytest.raises(tc.TcError) as e:
        tc.lang_dump(text, "sema")
    assert fragment in str(e.value)


@pytest.mark.parametrize("fragment,text", [
    ("", "def fun(float(M,N) A) -> (O) { O(i) +=! A(i,j) }"),
    ("", "def fun(float(M,N) A, float(M) B) -> (O) { O(i) = B(i) \n O(i) *= A(i,j) }"),
    ("", "def fun(float(M,N) A, float(M,N) B) -> (O) { O(i) max=! A(i,j) \n O(i) min= B(i,j) }"),
    ("+=! instead of +=", "def fun(float(M,N) A) -> (O) { O(i) += A(i,j) }"),
    ("*=! instead of *=", "def fun(float(M,N) A) -> (O) { O(i) *= A(i,j) }"),
    ("max=! instead of max=", "def fun(float(M,N) A) -> (O) { O(i) max= A(i,j) }"),
    ("min=! instead of min=", "def fun(float(M,N) A) -> (O) { O(i) min= A(i,j) }"),
])
def test_reduction_without_initialisation_warns(fragment, text):
    # with throw_warnings a warning becomes an exception, which makes it observable here
    tc.set_compiler_options(emit_warnings=False, throw_warnings=True)
    try:
        if fragment:
            with pytest.raises(tc.TcError) as e:
                tc.lang_dump(text, "sema")
            assert fragment in str(e.value)
        else:
            tc.lang_dump(text, "sema")
    finally:
        tc.set_compiler_options(True, False)


def test_canonical_form_ignores_names():
    one = """
    def fun(float(B, N, M) X, float(B, M, K) Y) -> (Z)
    {
       Z(b, i, j) += X(b, i, k) * Y(b, k, j)
    }
  """
    two = """
    def fun2(float(B, N, M) X, float(B, M, K) Y) -> (Q) {
            Q(b, ii, j) += X(b, ii, k) * Y(b, k, j)
    }
  """
    three = two.replace("Y(b, k, j)", "Y(b, j, k)")
    assert tc.lang_dump(one, "canonical") == tc.lang_dump(two, "canonical")
    assert tc.lang_dump(one, "canonical") != tc.lang_dump(three, "canonical")
