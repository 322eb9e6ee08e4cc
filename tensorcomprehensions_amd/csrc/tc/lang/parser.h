// Recursive-descent / precedence-climbing parser for TC.
//
// Grammar and operator precedences as in the reference parser (tc/lang/parser.h:23-318,
// precedence table tc/lang/lexer.h:138-151): ternary lowest and right-associative, then ||, &&,
// comparisons, + -, * / %, unary - !.  Number literals holding '.' or 'e' are float, all others
// int32 (parser.h:33-40).
#pragma once
#include "tc/lang/tree.h"

namespace lang {

class Parser {
 public:
  explicit Parser(const std::string& src) : L(src) {}

  TreeRef parseIdent() {
    Token t = L.expect(TK_IDENT);
    return Ident::create(t.range, t.text());
  }

  TreeRef parseConst() {
    Token t = L.expect(TK_NUMBER);
    std::string s = t.text();
    bool isFloat = s.find('.') != std::string::npos || s.find('e') != std::string::npos;
    return Tree::make(
        TK_CONST, t.range,
        {Tree::number(t.doubleValue()), Tree::make(isFloat ? TK_FLOAT : TK_INT32, t.range)});
  }

  TreeRef parseExp(int minPrec = 0) {
    TreeRef left;
    int k = L.cur().kind;
    if (k == '-' || k == '!') {
      SourceRange r = L.cur().range;
      L.next();
      left = Tree::make(k, r, {parseExp(kUnaryPrec)});
    } else {
      left = parsePrimary();
    }
    for (;;) {
      int op = L.cur().kind;
      int prec = binaryPrec(op);
      if (prec == 0 || prec <= minPrec) {
        break;
      }
      SourceRange r = L.cur().range;
      L.next();
      if (op == '?') {
        // right associative: the false branch may itself hold a ternary
        TreeRef yes = parseExp();
        L.expect(':');
        TreeRef no = parseExp(prec - 1);
        left = Tree::make('?', r, {left, yes, no});
      } else {
        // (the operand is parsed before the list is formed: an exception thrown while a braced
        // list is being built leaves its earlier elements undestroyed with GCC before 12)
        TreeRef right = parseExp(prec);
        left = Tree::make(op, r, {left, right});
      }
    }
    return left;
  }

  TreeRef parseStmt() {
    TreeRef ident = parseIdent();
    TreeRef indices = L.cur().kind == '(' ? parseList([&] { return parseIdent(); })
                                          : makeList(L.cur().range);
    TreeRef assign = parseAssignment();
    TreeRef rhs = parseExp();
    SourceRange eqRange = L.cur().range;
    TreeRef equivalent;
    if (L.nextIf(TK_EQUIVALENT)) {
      Token name = L.expect(TK_IDENT);
      TreeRef accesses = parseList([&] { return parseExp(); });
      equivalent = Tree::make(
          TK_OPTION, eqRange,
          {Tree::make(TK_EQUIVALENT, eqRange, {Tree::string(name.text()), accesses})});
    } else {
      equivalent = Tree::make(TK_OPTION, eqRange);
    }
    TreeRef where;
    if (L.nextIf(TK_WHERE)) {
      TreeList clauses;
      do {
        clauses.push_back(parseWhereClause());
      } while (L.nextIf(','));
      SourceRange whereRange = clauses.front()->range();
      where = makeList(whereRange, std::move(clauses));
    } else {
      where = makeList(L.cur().range);
    }
    TreeRef noReductions = makeList(ident->range());
    return Tree::make(
        TK_COMPREHENSION, ident->range(),
        {ident, indices, assign, rhs, where, equivalent, noReductions});
  }

  TreeRef parseFunction() {
    L.expect(TK_DEF);
    TreeRef name = parseIdent();
    TreeRef params = parseList([&] { return parseParam(); });
    L.expect(TK_ARROW);
    TreeRef returns = parseList([&] { return parseParam(); });
    L.expect('{');
    SourceRange r = L.cur().range;
    TreeList stmts;
    while (!L.nextIf('}')) {
      stmts.push_back(parseStmt());
    }
    return Tree::make(TK_DEF, name->range(), {name, params, returns, makeList(r, std::move(stmts))});
  }

  Lexer L;

 private:
  static constexpr int kUnaryPrec = 7;
  static int binaryPrec(int kind) {
    switch (kind) {
      case '?': return 1;
      case TK_OR: return 2;
      case TK_AND: return 3;
      case '>': case '<': case TK_LE: case TK_GE: case TK_EQ: case TK_NE: return 4;
      case '+': case '-': return 5;
      case '*': case '/': case '%': return 6;
      default: return 0;
    }
  }

  template <typename F>
  TreeRef parseList(F parseElement) {
    SourceRange r = L.cur().range;
    L.expect('(');
    TreeList elems;
    if (L.cur().kind != ')') {
      do {
        elems.push_back(parseElement());
      } while (L.nextIf(','));
    }
    L.expect(')');
    return makeList(r, std::move(elems));
  }

  TreeRef parsePrimary() {
    int k = L.cur().kind;
    if (k == TK_NUMBER) {
      return parseConst();
    }
    if (k == '(') {
      L.next();
      TreeRef e = parseExp();
      L.expect(')');
      return e;
    }
    if (isScalarTypeKind(k)) { // cast: float(x + 1)
      TreeRef type = parseScalarType();
      L.expect('(');
      TreeRef value = parseExp();
      L.expect(')');
      return Tree::make(TK_CAST, type->range(), {value, type});
    }
    if (k == TK_MIN || k == TK_MAX) { // two-argument operators spelled like calls
      SourceRange r = L.cur().range;
      L.next();
      L.expect('(');
      TreeRef a = parseExp();
      L.expect(',');
      TreeRef b = parseExp();
      L.expect(')');
      return Tree::make(k, r, {a, b});
    }
    TreeRef id = parseIdent();
    if (L.cur().kind == '(') {
      SourceRange r = L.cur().range;
      return Apply::create(TK_APPLY, r, id, parseList([&] { return parseExp(); }));
    }
    return id;
  }

  TreeRef parseScalarType() {
    if (!isScalarTypeKind(L.cur().kind)) {
      L.reportError("a scalar type");
    }
    Token t = L.next();
    return Tree::make(t.kind, t.range);
  }

  TreeRef parseType() {
    TreeRef scalar = parseScalarType();
    TreeRef dims = L.cur().kind == '('
        ? parseList([&] { return L.cur().kind == TK_NUMBER ? parseConst() : parseIdent(); })
        : makeList(L.cur().range);
    return TensorType::create(scalar->range(), scalar, dims);
  }

  TreeRef parseParam() {
    if (L.cur().kind == TK_IDENT) {
      TreeRef id = parseIdent();
      return Param::create(id->range(), id, Tree::make(TK_INFERRED, id->range()));
    }
    TreeRef type = parseType();
    TreeRef id = parseIdent();
    return Param::create(type->range(), id, type);
  }

  TreeRef parseAssignment() {
    switch (L.cur().kind) {
      case '=': case TK_PLUS_EQ: case TK_TIMES_EQ: case TK_MIN_EQ: case TK_MAX_EQ:
      case TK_PLUS_EQ_B: case TK_TIMES_EQ_B: case TK_MIN_EQ_B: case TK_MAX_EQ_B: {
        int kind = L.next().kind;
        return Tree::make(kind, L.cur().range);
      }
      default:
        L.reportError("a valid assignment operator");
    }
  }

  TreeRef parseWhereClause() {
    int ahead = L.lookahead().kind;
    if (ahead == '=') {
      TreeRef id = parseIdent();
      L.expect('=');
      TreeRef rhs = parseExp();
      return Tree::make(TK_LET, id->range(), {id, rhs});
    }
    if (ahead == TK_IN) {
      TreeRef id = parseIdent();
      L.expect(TK_IN);
      TreeRef lo = parseExp();
      L.expect(':');
      TreeRef hi = parseExp();
      return Tree::make(TK_RANGE_CONSTRAINT, id->range(), {id, lo, hi});
    }
    L.expect(TK_EXISTS);
    TreeRef e = parseExp();
    return Tree::make(TK_EXISTS, e->range(), {e});
  }
};

} // namespace lang
