// Lowering of a checked TC function to tc::ir with forward range inference on concrete sizes.
//
// Range inference restates tc/core/tc2halide.cc:270-498: every tensor access contributes
// "subscript within the tensor's bounds" inequalities; variables are solved round by round, a
// variable being solvable in a round when some inequalities mention no other unsolved variable;
// the solution is the largest interval satisfying them; solved variables are then eliminated
// from the remaining inequalities by their worst case.  `where i in a:b` fixes [a, b-1] up front
// (:652-669).  Reduction indices are the right-hand-side variables absent from the left-hand
// side, in order of first appearance (:698-740).  Because sizes are known here, intervals are
// numbers rather than symbolic expressions.
#include <algorithm>
#include <cmath>
#include <functional>
#include <limits>
#include <set>

#include "tc/core/check.h"
#include "tc/core/ir.h"
#include "tc/lang/sema.h"

namespace tc {
namespace ir {

Affine toAffine(const ExprRef& e) {
  Affine a;
  switch (e->kind) {
    case Expr::IntImm:
      a.valid = true;
      a.constant = e->ival;
      return a;
    case Expr::Var:
      a.valid = true;
      a.coef[e->name] = 1;
      return a;
    case Expr::Cast:
      if (!e->type.isFloat() && !e->args[0]->type.isFloat()) {
        return toAffine(e->args[0]);
      }
      return a;
    case Expr::Unary:
      if (e->name == "-") {
        Affine x = toAffine(e->args[0]);
        if (x.valid) {
          for (auto& c : x.coef) c.second = -c.second;
          x.constant = -x.constant;
        }
        return x;
      }
      return a;
    case Expr::Binary: {
      if (e->name != "+" && e->name != "-" && e->name != "*") {
        return a;
      }
      Affine x = toAffine(e->args[0]), y = toAffine(e->args[1]);
      if (!x.valid || !y.valid) {
        return a;
      }
      if (e->name == "*") {
        const Affine* k = x.coef.empty() ? &x : y.coef.empty() ? &y : nullptr;
        if (!k) {
          return a;
        }
        const Affine& o = (k == &x) ? y : x;
        a.valid = true;
        for (const auto& c : o.coef) {
          if (c.second * k->constant != 0) a.coef[c.first] = c.second * k->constant;
        }
        a.constant = o.constant * k->constant;
        return a;
      }
      int64_t sg = e->name == "+" ? 1 : -1;
      a = x;
      for (const auto& c : y.coef) {
        a.coef[c.first] += sg * c.second;
        if (a.coef[c.first] == 0) a.coef.erase(c.first);
      }
      a.constant += sg * y.constant;
      return a;
    }
    default:
      return a;
  }
}

std::string identityLiteral(ReduceOp op, const ScalarType& t) {
  if (t.isFloat() && t.bits == 16) {
    // largest finite half is 65504
    switch (op) {
      case ReduceOp::Times: return "((_Float16)1.0f)";
      case ReduceOp::Min: return "((_Float16)65504.0f)";
      case ReduceOp::Max: return "((_Float16)-65504.0f)";
      default: return "((_Float16)0.0f)";
    }
  }
  auto lit = [&](double v) -> std::string {
    std::ostringstream ss;
    if (t.isFloat()) {
      ss.precision(t.bits == 64 ? 17 : 9);
      ss << std::scientific << v << (t.bits == 32 ? "f" : "");
    } else {
      ss << static_cast<long long>(v);
    }
    return ss.str();
  };
  switch (op) {
    case ReduceOp::Plus:
    case ReduceOp::None:
      return t.isFloat() ? (t.bits == 32 ? "0.0f" : "0.0") : "0";
    case ReduceOp::Times:
      return t.isFloat() ? (t.bits == 32 ? "1.0f" : "1.0") : "1";
    case ReduceOp::Min:
    case ReduceOp::Max: {
      bool wantMax = op == ReduceOp::Min; // min starts from the type's maximum
      if (t.isFloat()) {
        double m = t.bits == 32 ? static_cast<double>(std::numeric_limits<float>::max())
                                : std::numeric_limits<double>::max();
        return lit(wantMax ? m : -m);
      }
      if (t.code == ScalarType::UInt) {
        if (!wantMax) return "0";
        return t.bits == 64 ? "18446744073709551615ULL" : std::to_string((1ULL << t.bits) - 1) + "U";
      }
      if (t.bits == 64) {
        return wantMax ? "9223372036854775807LL" : "(-9223372036854775807LL - 1)";
      }
      long long m = (1LL << (t.bits - 1)) - 1;
      return wantMax ? std::to_string(m) : "(" + std::to_string(-m) + " - 1)";
    }
  }
  return "0";
}

} // namespace ir

namespace tc2ir {
namespace {

using namespace ir;
using lang::TreeRef;

ScalarType scalarOf(const TreeRef& typeTree) {
  lang::TypeInfo ti(typeTree);
  ScalarType s;
  s.code = static_cast<ScalarType::Code>(ti.code);
  s.bits = ti.bits;
  return s;
}

ExprRef mk(Expr::Kind k, ScalarType t, std::string name = "", std::vector<ExprRef> args = {}) {
  auto e = std::make_shared<Expr>();
  e->kind = k;
  e->type = t;
  e->name = std::move(name);
  e->args = std::move(args);
  return e;
}
ExprRef intImm(int64_t v) {
  auto e = std::make_shared<Expr>();
  e->kind = Expr::IntImm;
  e->type = ScalarType{ScalarType::Int, 32};
  e->ival = v;
  return e;
}

// one "coef . vars + k >= 0" inequality, or an opaque one (non-affine subscript)
struct Ineq {
  bool opaque = false;
  std::map<std::string, int64_t> coef;
  int64_t k = 0;
  std::set<std::string> vars; // opaque only
};

struct Lowering {
  lang::Sema& sema;
  Function& f;
  const CompilerOptions& opts;
  std::map<std::string, std::map<std::string, Range>> boundsByName; // tensor -> index name -> range

  std::string opName(int kind) {
    switch (kind) {
      case lang::TK_EQ: return "==";
      case lang::TK_NE: return "!=";
      case lang::TK_LE: return "<=";
      case lang::TK_GE: return ">=";
      case lang::TK_AND: return "&&";
      case lang::TK_OR: return "||";
      case lang::TK_MIN: return "min";
      case lang::TK_MAX: return "max";
      default: return std::string(1, static_cast<char>(kind));
    }
  }

  ExprRef lower(const TreeRef& e, const std::map<std::string, ExprRef>& lets) {
    auto sub = [&](size_t i) { return lower(e->tree(i), lets); };
    switch (e->kind()) {
      case lang::TK_IDENT: {
        const std::string& n = lang::Ident(e).name();
        auto l = lets.find(n);
        if (l != lets.end()) {
          return l->second;
        }
        auto p = f.params.find(n);
        if (p != f.params.end()) {
          return intImm(p->second);
        }
        return mk(Expr::Var, ScalarType{ScalarType::Int, 32}, n);
      }
      case lang::TK_ACCESS: {
        lang::Apply a(e);
        std::vector<ExprRef> args;
        for (const auto& x : a.arguments()) {
          args.push_back(lower(x, lets));
        }
        return mk(Expr::Load, scalarOf(sema.typeOfExpr(e)), a.name().name(), std::move(args));
      }
      case lang::TK_BUILT_IN: {
        lang::BuiltIn b(e);
        std::vector<ExprRef> args;
        for (const auto& x : b.arguments()) {
          args.push_back(lower(x, lets));
        }
        return mk(Expr::Call, scalarOf(b.type()), b.name(), std::move(args));
      }
      case lang::TK_CONST: {
        lang::Const c(e);
        auto x = std::make_shared<Expr>();
        x->type = scalarOf(c.type());
        if (x->type.isFloat()) {
          x->kind = Expr::FloatImm;
          x->fval = static_cast<float>(c.value());
        } else {
          x->kind = Expr::IntImm;
          x->ival = static_cast<int64_t>(c.value());
        }
        return x;
      }
      case lang::TK_CAST:
        return mk(Expr::Cast, scalarOf(lang::Cast(e).type()), "", {lower(lang::Cast(e).value(), lets)});
      case '?':
      {
        // (operands first, the list after: see lang::Parser::parseExp)
        ExprRef cond = sub(0), yes = sub(1), no = sub(2);
        return mk(Expr::Select, scalarOf(sema.typeOfExpr(e)), "?", {cond, yes, no});
      }
      case '-':
        if (e->trees().size() == 1) {
          return mk(Expr::Unary, scalarOf(sema.typeOfExpr(e)), "-", {sub(0)});
        }
        // fallthrough
      case '+': case '*': case '/': case '%': case lang::TK_MIN: case lang::TK_MAX:
      case lang::TK_EQ: case lang::TK_NE: case lang::TK_LE: case lang::TK_GE: case '<': case '>':
      case lang::TK_AND: case lang::TK_OR:
      {
        ExprRef left = sub(0), right = sub(1);
        return mk(Expr::Binary, scalarOf(sema.typeOfExpr(e)), opName(e->kind()), {left, right});
      }
      case '!':
        return mk(Expr::Unary, scalarOf(sema.typeOfExpr(e)), "!", {sub(0)});
      default:
        throw lang::errorAt(e) << "Unhandled TC expr: " << lang::kindToString(e->kind());
    }
  }

  // variables in order of first appearance
  void varsOf(const ExprRef& e, std::vector<std::string>& out) {
    if (e->kind == Expr::Var && std::find(out.begin(), out.end(), e->name) == out.end()) {
      out.push_back(e->name);
    }
    for (const auto& a : e->args) {
      varsOf(a, out);
    }
  }

  void collect(const ExprRef& e, std::vector<Ineq>& ineqs) {
    for (const auto& a : e->args) {
      collect(a, ineqs);
    }
    if (e->kind != Expr::Load) {
      return;
    }
    const Tensor* t = f.find(e->name);
    TC_CHECK(t) << "access to unknown tensor " << e->name;
    for (size_t d = 0; d < e->args.size(); ++d) {
      int64_t lo = t->mins[d], hi = t->mins[d] + t->extents[d] - 1;
      Affine a = toAffine(e->args[d]);
      if (!a.valid) {
        Ineq q;
        q.opaque = true;
        std::vector<std::string> vs;
        varsOf(e->args[d], vs);
        q.vars.insert(vs.begin(), vs.end());
        ineqs.push_back(q);
        continue;
      }
      Ineq ge, le;
      ge.coef = a.coef;
      ge.k = a.constant - lo; // subscript - lo >= 0
      for (const auto& c : a.coef) {
        le.coef[c.first] = -c.second;
      }
      le.k = hi - a.constant; // hi - subscript >= 0
      ineqs.push_back(ge);
      ineqs.push_back(le);
    }
  }

  static int64_t floorDiv(int64_t a, int64_t b) {
    int64_t q = a / b;
    return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
  }

  void solve(const TreeRef& stmtTree, std::vector<Ineq> ineqs, const std::vector<std::string>& freeVars,
             std::map<std::string, Range>& solution) {
    auto warnUnchecked = [&](const std::string& what) {
      lang::ErrorReport w(stmtTree->range());
      w << "Required precondition will not be checked at runtime: " << what;
      if (opts.throwWarnings) {
        throw w;
      }
      f.warnings.push_back(w.message());
      if (opts.emitWarnings) {
        std::cerr << "WARNING: " << w.what();
      }
    };
    // worst case of every inequality over the solved variables; inequalities left without
    // variables are dropped (with a warning when they do not hold)
    auto eliminate = [&]() {
      std::vector<Ineq> kept;
      for (auto& q : ineqs) {
        if (q.opaque) {
          for (auto it = q.vars.begin(); it != q.vars.end();) {
            it = solution.count(*it) ? q.vars.erase(it) : std::next(it);
          }
          if (q.vars.empty()) {
            warnUnchecked("a non-affine subscript stays within its tensor");
          } else {
            kept.push_back(q);
          }
          continue;
        }
        bool hadVars = !q.coef.empty();
        for (auto it = q.coef.begin(); it != q.coef.end();) {
          auto s = solution.find(it->first);
          if (s == solution.end()) {
            ++it;
            continue;
          }
          q.k += it->second * (it->second > 0 ? s->second.min : s->second.max);
          it = q.coef.erase(it);
        }
        if (q.coef.empty()) {
          if (q.k < 0 && hadVars) {
            warnUnchecked("an access is out of bounds for part of the inferred ranges");
          } else if (q.k < 0) {
            warnUnchecked("a constant subscript is out of bounds");
          }
        } else {
          kept.push_back(q);
        }
      }
      ineqs.swap(kept);
    };

    std::set<std::string> unsolved;
    for (const auto& v : freeVars) {
      if (!solution.count(v)) {
        unsolved.insert(v);
      }
    }
    eliminate();
    while (!unsolved.empty()) {
      std::set<std::string> still;
      for (const auto& v : unsolved) {
        bool hasLo = false, hasHi = false;
        int64_t lo = 0, hi = 0;
        std::vector<Ineq> rest;
        for (const auto& q : ineqs) {
          if (q.opaque || q.coef.size() != 1 || q.coef.begin()->first != v) {
            rest.push_back(q);
            continue;
          }
          int64_t a = q.coef.begin()->second;
          if (a > 0) { // a v + k >= 0  ->  v >= ceil(-k / a)
            int64_t b = -floorDiv(q.k, a);
            lo = hasLo ? std::max(lo, b) : b;
            hasLo = true;
          } else { // v <= floor(k / -a)
            int64_t b = floorDiv(q.k, -a);
            hi = hasHi ? std::min(hi, b) : b;
            hasHi = true;
          }
        }
        if (hasLo && hasHi && lo > hi) {
          throw lang::errorAt(stmtTree) << "Inferred an empty range for variable " << v;
        }
        if (!hasLo || !hasHi) {
          still.insert(v);
        } else {
          solution[v] = Range{lo, hi};
          ineqs.swap(rest);
        }
      }
      eliminate();
      if (still.size() == unsolved.size()) {
        lang::ErrorReport err(stmtTree->range());
        for (const auto& v : unsolved) {
          err << "Unsolved variable: " << v << '\n';
        }
        err << "Could not infer ranges for free variables. Use a where clause";
        throw err;
      }
      unsolved.swap(still);
    }
  }

  int64_t constantOf(const ExprRef& e, const TreeRef& where) {
    Affine a = toAffine(e);
    if (!a.valid || !a.coef.empty()) {
      throw lang::errorAt(where) << "range bounds must be integer expressions of the size parameters";
    }
    return a.constant;
  }

  void lowerStatement(const TreeRef& stmtTree) {
    lang::Comprehension c(stmtTree);
    Statement s;
    s.tree = stmtTree;
    s.tensor = c.ident().name();
    for (const auto& i : c.indices()) {
      s.lhsVars.push_back(lang::Ident(i).name());
    }
    std::map<std::string, ExprRef> lets;
    std::map<std::string, Range> solution;
    std::vector<ExprRef> existsExprs;
    for (const auto& w : c.whereClauses()) {
      if (w->kind() == lang::TK_LET) {
        lang::Let l(w);
        lets[l.name().name()] = lower(l.rhs(), lets);
      }
    }
    for (const auto& w : c.whereClauses()) {
      if (w->kind() == lang::TK_RANGE_CONSTRAINT) {
        lang::RangeConstraint rc(w);
        int64_t lo = constantOf(lower(rc.start(), lets), rc.start());
        int64_t hi = constantOf(lower(rc.end(), lets), rc.end()) - 1; // [a, b)
        solution[rc.ident().name()] = Range{lo, hi};
      } else if (w->kind() == lang::TK_EXISTS) {
        existsExprs.push_back(lower(w->tree(0), lets));
      }
    }
    s.rhs = lower(c.rhs(), lets);
    s.type = s.rhs->type;
    switch (c.assignment()->kind()) {
      case '=': s.op = ReduceOp::None; break;
      case lang::TK_PLUS_EQ_B: s.init = true; // fallthrough
      case lang::TK_PLUS_EQ: s.op = ReduceOp::Plus; break;
      case lang::TK_TIMES_EQ_B: s.init = true; // fallthrough
      case lang::TK_TIMES_EQ: s.op = ReduceOp::Times; break;
      case lang::TK_MIN_EQ_B: s.init = true; // fallthrough
      case lang::TK_MIN_EQ: s.op = ReduceOp::Min; break;
      case lang::TK_MAX_EQ_B: s.init = true; // fallthrough
      case lang::TK_MAX_EQ: s.op = ReduceOp::Max; break;
      default:
        throw lang::errorAt(stmtTree) << "Unimplemented reduction " << c.assignment()->range().text();
    }

    std::vector<Ineq> ineqs;
    std::vector<std::string> freeVars;
    for (const auto& e : existsExprs) {
      collect(e, ineqs);
      varsOf(e, freeVars);
    }
    collect(s.rhs, ineqs);
    varsOf(s.rhs, freeVars);
    solve(stmtTree, ineqs, freeVars, solution);

    for (const auto& v : s.lhsVars) {
      if (!solution.count(v)) {
        throw lang::errorAt(stmtTree) << "Free variable " << v
                                      << " was not solved in range inference. May not be used right-hand side";
      }
    }
    std::vector<std::string> order;
    varsOf(s.rhs, order);
    for (const auto& v : order) {
      if (std::find(s.lhsVars.begin(), s.lhsVars.end(), v) == s.lhsVars.end()) {
        if (!solution.count(v)) {
          throw lang::errorAt(stmtTree) << "Free variable " << v
                                        << " is unconstrained. Use a 'where' clause to set its range.";
        }
        s.redVars.push_back(v);
      }
    }
    for (const auto& v : s.lhsVars) s.ranges[v] = solution[v];
    for (const auto& v : s.redVars) s.ranges[v] = solution[v];
    if (s.redVars.empty() && s.init) {
      // "op=!" without reduction indices: initialise then combine once == plain assignment
      s.op = ReduceOp::None;
      s.init = false;
    }

    // record (or clobber) the written tensor's bounds
    Tensor* out = nullptr;
    for (auto& t : f.outputs) {
      if (t.name == s.tensor) out = &t;
    }
    TC_CHECK(out) << s.tensor << " is not an output";
    if (!(out->argNames.empty() && out->extents.empty())) {
      // a later statement of a tensor keeps the type of its first definition; Halide refuses an
      // update definition of another type, so a value that would lose precision is an error
      // here as it is for outputs annotated with a type (sema.h:531-551)
      const ScalarType &have = out->type, &got = s.type;
      bool narrows = (got.code == ScalarType::Float && have.code != ScalarType::Float) ||
          (got.code == have.code && got.bits > have.bits);
      if (narrows) {
        throw lang::errorAt(stmtTree) << " attempting to assign type " << got.cName() << " to narrower type "
                                      << have.cName() << " without an explicit cast";
      }
    }
    if (out->argNames.empty() && out->extents.empty()) {
      out->argNames = s.lhsVars;
      out->type = s.type;
      out->mins.assign(s.lhsVars.size(), 0);
      out->extents.assign(s.lhsVars.size(), 0);
      defined_.insert(s.tensor);
    }
    auto& byName = boundsByName[s.tensor];
    for (const auto& v : s.lhsVars) {
      byName[v] = solution[v];
    }
    for (size_t d = 0; d < out->argNames.size(); ++d) {
      const Range& r = byName.at(out->argNames[d]);
      out->mins[d] = r.min;
      out->extents[d] = r.extent();
    }
    defined_.insert(s.tensor);
    f.statements.push_back(std::move(s));
  }

  std::set<std::string> defined_;
};

} // namespace

ir::Function translate(
    const lang::TreeRef& defTree,
    const std::vector<std::vector<int64_t>>& inputShapes,
    const CompilerOptions& options) {
  lang::Sema sema(options);
  TreeRef checked = sema.checkFunction(defTree);
  lang::Def def(checked);
  ir::Function f;
  f.name = def.name().name();
  f.def = checked;
  if (def.params().size() != inputShapes.size()) {
    throw lang::errorAt(checked) << "expected " << def.params().size() << " inputs but got "
                                 << inputShapes.size();
  }
  for (size_t i = 0; i < def.params().size(); ++i) {
    lang::Param p(def.params()[i]);
    lang::TensorType tt = p.tensorType();
    const auto& shape = inputShapes[i];
    if (tt.dims().size() != shape.size()) {
      throw lang::errorAt(def.params()[i]) << "expected a tensor with " << tt.dims().size()
                                           << " dimensions but found " << shape.size() << " dimensions.";
    }
    ir::Tensor t;
    t.name = p.ident().name();
    t.type = scalarOf(tt.scalarTypeTree());
    t.isInput = true;
    for (size_t d = 0; d < shape.size(); ++d) {
      const TreeRef& dim = tt.dims()[d];
      if (dim->kind() == lang::TK_IDENT) {
        const std::string& n = lang::Ident(dim).name();
        auto it = f.params.find(n);
        if (it != f.params.end() && it->second != shape[d]) {
          throw lang::errorAt(dim) << "Mismatched sizes for dimension " << n << " previous value is "
                                   << it->second << " but found " << shape[d] << " here";
        }
        f.params[n] = shape[d];
      } else {
        int64_t c = static_cast<int64_t>(lang::Const(dim).value());
        if (c != shape[d]) {
          throw lang::errorAt(dim) << "Constant dimension expected size " << c << " but found " << shape[d];
        }
      }
      t.mins.push_back(0);
      t.extents.push_back(shape[d]);
    }
    f.inputs.push_back(std::move(t));
  }
  for (const auto& r : def.returns()) {
    ir::Tensor t;
    t.name = lang::Param(r).ident().name();
    f.outputs.push_back(std::move(t));
  }
  Lowering L{sema, f, options, {}, {}};
  for (const auto& s : def.statements()) {
    L.lowerStatement(s);
  }
  for (const auto& o : f.outputs) {
    if (!L.defined_.count(o.name)) {
      throw lang::errorAt(checked) << "output " << o.name << " is never written";
    }
  }
  // A tensor has one bound, that of its last definition, applied to all its stages
  // (tc2halide.cc:676-693, :808-870): an earlier statement inferred over a larger range writes
  // only inside it.
  for (auto& s : f.statements) {
    const ir::Tensor* out = nullptr;
    for (const auto& t : f.outputs) {
      if (t.name == s.tensor) out = &t;
    }
    for (size_t d = 0; d < s.lhsVars.size() && d < out->extents.size(); ++d) {
      ir::Range& r = s.ranges[s.lhsVars[d]];
      r.min = std::max(r.min, out->mins[d]);
      r.max = std::min(r.max, out->mins[d] + out->extents[d] - 1);
    }
  }
  return f;
}

} // namespace tc2ir
} // namespace tc
