// Range inference on symbolic sizes: the solver of tc2ir.cc (tc/core/tc2halide.cc:270-498 in the
// reference) with linear forms over size parameters where that one has numbers.
#include "tc/core/symbolic_ranges.h"

#include <algorithm>
#include <set>
#include <sstream>

#include "tc/core/check.h"
#include "tc/lang/sema.h"

namespace tc {
namespace symbolic {
namespace {

using lang::TreeRef;

int64_t floorDivInt(int64_t a, int64_t b) {
  int64_t q = a / b;
  return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
}

Lin constant(int64_t v) {
  Lin l;
  l.k = v;
  return l;
}
Lin scaled(const Lin& a, int64_t s) {
  Lin r;
  if (s == 0) return r;
  for (const auto& c : a.coef) r.coef[c.first] = c.second * s;
  r.k = a.k * s;
  return r;
}
Lin sum(const Lin& a, const Lin& b) {
  Lin r = a;
  for (const auto& c : b.coef) {
    int64_t& x = r.coef[c.first];
    x += c.second;
    if (x == 0) r.coef.erase(c.first);
  }
  r.k += b.k;
  return r;
}
Lin difference(const Lin& a, const Lin& b) { return sum(a, scaled(b, -1)); }

// one "coef . vars + k >= 0" inequality over index variables, or an opaque one
struct Ineq {
  bool opaque = false;
  std::map<std::string, int64_t> coef;
  Lin k;
  std::set<std::string> vars; // opaque only
};

// an index expression: integer coefficients on index variables, the rest a linear form of sizes
struct IndexAffine {
  bool valid = false;
  std::map<std::string, int64_t> coef;
  Lin k;
};

struct Solver {
  FunctionRanges& out;
  std::set<std::string> paramNames;
  std::map<std::string, TensorBounds*> tensors;
  std::map<std::string, std::map<std::string, Range>> boundsByName;

  // ---- atoms -------------------------------------------------------------------------------
  Lin atom(const Atom& a, const std::string& key) {
    out.atoms.emplace(key, a);
    Lin l;
    l.coef[key] = 1;
    return l;
  }
  Lin param(const std::string& name) {
    Atom a;
    a.kind = Atom::Param;
    return atom(a, name);
  }
  Lin extremum(Atom::Kind kind, const Lin& a, const Lin& b) {
    Lin d = difference(a, b);
    if (d.isConstant()) {
      const bool first = kind == Atom::Max ? d.k >= 0 : d.k <= 0;
      return first ? a : b;
    }
    std::string ta = out.text(a), tb = out.text(b);
    Atom n;
    n.kind = kind;
    const bool swap = tb < ta;
    n.a = swap ? b : a;
    n.b = swap ? a : b;
    if (swap) std::swap(ta, tb);
    return atom(n, std::string(kind == Atom::Max ? "max(" : "min(") + ta + ", " + tb + ")");
  }
  // floor(a / d), d > 0: the part of `a` divisible by d leaves the division
  Lin floorDiv(const Lin& a, int64_t d) {
    TC_CHECK_GT(d, 0);
    if (d == 1) return a;
    Lin q, r;
    // floor((d X + R) / d) = X + floor(R / d) for any integer X: coefficients are split by
    // truncation, so that what stays under the division reads like what was written
    for (const auto& c : a.coef) {
      const int64_t whole = c.second / d, rest = c.second - whole * d;
      if (whole != 0) q.coef[c.first] = whole;
      if (rest != 0) r.coef[c.first] = rest;
    }
    const int64_t whole = a.k / d;
    q.k = whole;
    r.k = a.k - whole * d;
    if (r.isConstant()) {
      q.k += floorDivInt(r.k, d);
      return q;
    }
    Atom n;
    n.kind = Atom::FloorDiv;
    n.a = r;
    n.d = d;
    return sum(q, atom(n, "((" + out.text(r) + ") // " + std::to_string(d) + ")"));
  }

  // ---- expressions -------------------------------------------------------------------------
  IndexAffine affineOf(const TreeRef& e, const std::map<std::string, TreeRef>& lets) {
    IndexAffine a;
    switch (e->kind()) {
      case lang::TK_IDENT: {
        const std::string& n = lang::Ident(e).name();
        auto l = lets.find(n);
        if (l != lets.end()) return affineOf(l->second, lets);
        a.valid = true;
        if (paramNames.count(n)) {
          a.k = param(n);
        } else {
          a.coef[n] = 1;
        }
        return a;
      }
      case lang::TK_CONST: {
        lang::Const c(e);
        const double v = c.value();
        if (v != static_cast<double>(static_cast<int64_t>(v))) return a;
        a.valid = true;
        a.k = constant(static_cast<int64_t>(v));
        return a;
      }
      case lang::TK_CAST:
        return affineOf(lang::Cast(e).value(), lets);
      case '-':
        if (e->trees().size() == 1) {
          IndexAffine x = affineOf(e->tree(0), lets);
          if (!x.valid) return a;
          for (auto& c : x.coef) c.second = -c.second;
          x.k = scaled(x.k, -1);
          return x;
        }
        // fallthrough
      case '+': {
        IndexAffine x = affineOf(e->tree(0), lets), y = affineOf(e->tree(1), lets);
        if (!x.valid || !y.valid) return a;
        const int64_t sg = e->kind() == '+' ? 1 : -1;
        a = x;
        for (const auto& c : y.coef) {
          int64_t& v = a.coef[c.first];
          v += sg * c.second;
          if (v == 0) a.coef.erase(c.first);
        }
        a.k = sum(x.k, scaled(y.k, sg));
        return a;
      }
      case '*': {
        IndexAffine x = affineOf(e->tree(0), lets), y = affineOf(e->tree(1), lets);
        if (!x.valid || !y.valid) return a;
        const bool xConst = x.coef.empty() && x.k.isConstant(), yConst = y.coef.empty() && y.k.isConstant();
        if (!xConst && !yConst) return a;
        const IndexAffine& o = xConst ? y : x;
        const int64_t s = xConst ? x.k.k : y.k.k;
        a.valid = true;
        for (const auto& c : o.coef) {
          if (c.second * s != 0) a.coef[c.first] = c.second * s;
        }
        a.k = scaled(o.k, s);
        return a;
      }
      default:
        return a;
    }
  }

  void indexVarsOf(const TreeRef& e, const std::map<std::string, TreeRef>& lets, std::vector<std::string>& vars) {
    if (e->kind() == lang::TK_IDENT) {
      const std::string& n = lang::Ident(e).name();
      auto l = lets.find(n);
      if (l != lets.end()) {
        indexVarsOf(l->second, lets, vars);
      } else if (!paramNames.count(n) && !tensors.count(n) && std::find(vars.begin(), vars.end(), n) == vars.end()) {
        vars.push_back(n);
      }
      return;
    }
    if (e->kind() == lang::TK_ACCESS) {
      for (const auto& x : lang::Apply(e).arguments()) indexVarsOf(x, lets, vars);
      return;
    }
    if (e->kind() == lang::TK_BUILT_IN) {
      for (const auto& x : lang::BuiltIn(e).arguments()) indexVarsOf(x, lets, vars);
      return;
    }
    if (e->kind() == lang::TK_CONST) return;
    if (e->kind() == lang::TK_CAST) {
      indexVarsOf(lang::Cast(e).value(), lets, vars);
      return;
    }
    for (const auto& t : e->trees()) indexVarsOf(t, lets, vars);
  }

  void collect(const TreeRef& e, const std::map<std::string, TreeRef>& lets, std::vector<Ineq>& ineqs) {
    if (e->kind() == lang::TK_IDENT) {
      auto l = lets.find(lang::Ident(e).name());
      if (l != lets.end()) collect(l->second, lets, ineqs);
      return;
    }
    if (e->kind() == lang::TK_CONST) return;
    if (e->kind() == lang::TK_CAST) {
      collect(lang::Cast(e).value(), lets, ineqs);
      return;
    }
    if (e->kind() == lang::TK_BUILT_IN) {
      for (const auto& x : lang::BuiltIn(e).arguments()) collect(x, lets, ineqs);
      return;
    }
    if (e->kind() != lang::TK_ACCESS) {
      for (const auto& t : e->trees()) collect(t, lets, ineqs);
      return;
    }
    lang::Apply a(e);
    for (const auto& x : a.arguments()) collect(x, lets, ineqs);
    auto t = tensors.find(a.name().name());
    if (t == tensors.end()) throw lang::errorAt(e) << "access to unknown tensor " << a.name().name();
    const TensorBounds& b = *t->second;
    for (size_t d = 0; d < a.arguments().size() && d < b.mins.size(); ++d) {
      const Lin lo = b.mins[d], hi = sum(sum(b.mins[d], b.extents[d]), constant(-1));
      IndexAffine x = affineOf(a.arguments()[d], lets);
      if (!x.valid) {
        Ineq q;
        q.opaque = true;
        std::vector<std::string> vs;
        indexVarsOf(a.arguments()[d], lets, vs);
        q.vars.insert(vs.begin(), vs.end());
        ineqs.push_back(q);
        continue;
      }
      Ineq ge, le;
      ge.coef = x.coef;
      ge.k = difference(x.k, lo); // subscript - lo >= 0
      for (const auto& c : x.coef) le.coef[c.first] = -c.second;
      le.k = difference(hi, x.k); // hi - subscript >= 0
      ineqs.push_back(ge);
      ineqs.push_back(le);
    }
  }

  void solve(const TreeRef& stmt, std::vector<Ineq> ineqs, const std::vector<std::string>& freeVars,
             std::map<std::string, Range>& solution) {
    auto eliminate = [&]() {
      std::vector<Ineq> kept;
      for (auto& q : ineqs) {
        if (q.opaque) {
          for (auto it = q.vars.begin(); it != q.vars.end();) {
            it = solution.count(*it) ? q.vars.erase(it) : std::next(it);
          }
          if (!q.vars.empty()) kept.push_back(q);
          continue;
        }
        for (auto it = q.coef.begin(); it != q.coef.end();) {
          auto s = solution.find(it->first);
          if (s == solution.end()) {
            ++it;
            continue;
          }
          q.k = sum(q.k, scaled(it->second > 0 ? s->second.min : s->second.max, it->second));
          it = q.coef.erase(it);
        }
        if (!q.coef.empty()) kept.push_back(q);
      }
      ineqs.swap(kept);
    };
    std::set<std::string> unsolved;
    for (const auto& v : freeVars) {
      if (!solution.count(v)) unsolved.insert(v);
    }
    eliminate();
    while (!unsolved.empty()) {
      std::set<std::string> still;
      for (const auto& v : unsolved) {
        bool hasLo = false, hasHi = false;
        Lin lo, hi;
        std::vector<Ineq> rest;
        for (const auto& q : ineqs) {
          if (q.opaque || q.coef.size() != 1 || q.coef.begin()->first != v) {
            rest.push_back(q);
            continue;
          }
          const int64_t a = q.coef.begin()->second;
          if (a > 0) { // a v + k >= 0  ->  v >= -floor(k / a)
            Lin b = scaled(floorDiv(q.k, a), -1);
            lo = hasLo ? extremum(Atom::Max, lo, b) : b;
            hasLo = true;
          } else { // v <= floor(k / -a)
            Lin b = floorDiv(q.k, -a);
            hi = hasHi ? extremum(Atom::Min, hi, b) : b;
            hasHi = true;
          }
        }
        if (hasLo && hasHi) {
          Lin d = difference(hi, lo);
          if (d.isConstant() && d.k < 0) throw lang::errorAt(stmt) << "Inferred an empty range for variable " << v;
          solution[v] = Range{lo, hi};
          ineqs.swap(rest);
        } else {
          still.insert(v);
        }
      }
      eliminate();
      if (still.size() == unsolved.size()) {
        lang::ErrorReport err(stmt->range());
        for (const auto& v : unsolved) err << "Unsolved variable: " << v << '\n';
        err << "Could not infer ranges for free variables. Use a where clause";
        throw err;
      }
      unsolved.swap(still);
    }
  }

  Lin sizeExpression(const TreeRef& e, const std::map<std::string, TreeRef>& lets) {
    IndexAffine a = affineOf(e, lets);
    if (!a.valid || !a.coef.empty()) {
      throw lang::errorAt(e) << "range bounds must be integer expressions of the size parameters";
    }
    return a.k;
  }

  void statement(const TreeRef& stmtTree) {
    lang::Comprehension c(stmtTree);
    StatementRanges s;
    s.tensor = c.ident().name();
    std::vector<std::string> lhs;
    for (const auto& i : c.indices()) lhs.push_back(lang::Ident(i).name());
    std::map<std::string, TreeRef> lets;
    std::map<std::string, Range> solution;
    std::vector<TreeRef> exists;
    for (const auto& w : c.whereClauses()) {
      if (w->kind() == lang::TK_LET) {
        lang::Let l(w);
        lets[l.name().name()] = l.rhs();
      }
    }
    for (const auto& w : c.whereClauses()) {
      if (w->kind() == lang::TK_RANGE_CONSTRAINT) {
        lang::RangeConstraint rc(w);
        solution[rc.ident().name()] =
            Range{sizeExpression(rc.start(), lets), sum(sizeExpression(rc.end(), lets), constant(-1))}; // [a, b)
      } else if (w->kind() == lang::TK_EXISTS) {
        exists.push_back(w->tree(0));
      }
    }
    std::vector<Ineq> ineqs;
    std::vector<std::string> freeVars;
    for (const auto& e : exists) {
      collect(e, lets, ineqs);
      indexVarsOf(e, lets, freeVars);
    }
    collect(c.rhs(), lets, ineqs);
    indexVarsOf(c.rhs(), lets, freeVars);
    solve(stmtTree, ineqs, freeVars, solution);
    for (const auto& v : lhs) {
      if (!solution.count(v)) {
        throw lang::errorAt(stmtTree) << "Free variable " << v
                                      << " was not solved in range inference. May not be used right-hand side";
      }
      s.vars.emplace_back(v, solution[v]);
    }
    std::vector<std::string> order;
    indexVarsOf(c.rhs(), lets, order);
    for (const auto& v : order) {
      if (std::find(lhs.begin(), lhs.end(), v) != lhs.end()) continue;
      if (!solution.count(v)) {
        throw lang::errorAt(stmtTree) << "Free variable " << v << " is unconstrained. Use a 'where' clause to set its range.";
      }
      s.vars.emplace_back(v, solution[v]);
    }
    // record (or clobber) the written tensor's bounds: those of its last definition, by index name
    TensorBounds* t = tensors.at(s.tensor);
    auto& byName = boundsByName[s.tensor];
    if (argNames[s.tensor].empty() && t->mins.empty()) {
      argNames[s.tensor] = lhs;
      t->mins.assign(lhs.size(), Lin());
      t->extents.assign(lhs.size(), Lin());
    }
    for (const auto& v : lhs) byName[v] = solution[v];
    const auto& names = argNames[s.tensor];
    for (size_t d = 0; d < names.size(); ++d) {
      auto r = byName.find(names[d]);
      if (r == byName.end()) continue;
      t->mins[d] = r->second.min;
      t->extents[d] = sum(difference(r->second.max, r->second.min), constant(1));
    }
    out.statements.push_back(std::move(s));
  }

  std::map<std::string, std::vector<std::string>> argNames;
};

} // namespace

std::string FunctionRanges::text(const Lin& e) const {
  std::ostringstream ss;
  bool first = true;
  // size parameters in their order of appearance, other atoms after them by key
  std::vector<std::string> keys;
  for (const auto& p : params) {
    if (e.coef.count(p)) keys.push_back(p);
  }
  for (const auto& c : e.coef) {
    if (std::find(keys.begin(), keys.end(), c.first) == keys.end()) keys.push_back(c.first);
  }
  for (const auto& key : keys) {
    const int64_t c = e.coef.at(key);
    const int64_t mag = c < 0 ? -c : c;
    if (first) {
      if (c < 0) ss << "-";
    } else {
      ss << (c < 0 ? " - " : " + ");
    }
    if (mag != 1) ss << mag << "*";
    ss << key;
    first = false;
  }
  if (first) {
    ss << e.k;
  } else if (e.k != 0) {
    ss << (e.k < 0 ? " - " : " + ") << (e.k < 0 ? -e.k : e.k);
  }
  return ss.str();
}

int64_t FunctionRanges::evaluate(const Lin& e, const std::map<std::string, int64_t>& sizes) const {
  int64_t v = e.k;
  for (const auto& c : e.coef) {
    const Atom& a = atoms.at(c.first);
    int64_t x = 0;
    switch (a.kind) {
      case Atom::Param: {
        auto s = sizes.find(c.first);
        TC_CHECK(s != sizes.end()) << "no value for size parameter " << c.first;
        x = s->second;
        break;
      }
      case Atom::FloorDiv: x = floorDivInt(evaluate(a.a, sizes), a.d); break;
      case Atom::Min: x = std::min(evaluate(a.a, sizes), evaluate(a.b, sizes)); break;
      case Atom::Max: x = std::max(evaluate(a.a, sizes), evaluate(a.b, sizes)); break;
    }
    v += c.second * x;
  }
  return v;
}

std::string FunctionRanges::dump() const {
  std::ostringstream ss;
  auto block = [&](bool mins) {
    for (const auto* list : {&inputs, &outputs}) {
      for (const auto& t : *list) {
        ss << t.name << "@[";
        for (const auto& e : (mins ? t.mins : t.extents)) ss << text(e) << "; ";
        ss << "]\n";
      }
    }
  };
  ss << "mins:\n";
  block(true);
  ss << "extents:\n";
  block(false);
  return ss.str();
}

FunctionRanges inferRanges(const lang::TreeRef& defTree, const CompilerOptions& options) {
  lang::Sema sema(options);
  TreeRef checked = sema.checkFunction(defTree);
  lang::Def def(checked);
  FunctionRanges f;
  f.name = def.name().name();
  Solver s{f, {}, {}, {}, {}};
  // size parameters first: a dimension named like an earlier one is that size again
  for (const auto& p : def.params()) {
    lang::TensorType tt = lang::Param(p).tensorType();
    for (const auto& dim : tt.dims()) {
      if (dim->kind() != lang::TK_IDENT) continue;
      const std::string& n = lang::Ident(dim).name();
      if (s.paramNames.insert(n).second) f.params.push_back(n);
    }
  }
  f.inputs.reserve(def.params().size());
  f.outputs.reserve(def.returns().size());
  for (const auto& p : def.params()) {
    lang::Param param(p);
    lang::TensorType tt = param.tensorType();
    TensorBounds t;
    t.name = param.ident().name();
    for (const auto& dim : tt.dims()) {
      t.mins.push_back(Lin());
      if (dim->kind() == lang::TK_IDENT) {
        t.extents.push_back(s.param(lang::Ident(dim).name()));
      } else {
        t.extents.push_back(constant(static_cast<int64_t>(lang::Const(dim).value())));
      }
    }
    f.inputs.push_back(std::move(t));
  }
  for (const auto& r : def.returns()) {
    TensorBounds t;
    t.name = lang::Param(r).ident().name();
    f.outputs.push_back(std::move(t));
  }
  for (auto& t : f.inputs) s.tensors[t.name] = &t;
  for (auto& t : f.outputs) s.tensors[t.name] = &t;
  for (const auto& st : def.statements()) s.statement(st);
  for (const auto& o : f.outputs) {
    if (o.mins.empty() && !s.argNames.count(o.name)) {
      throw lang::errorAt(checked) << "output " << o.name << " is never written";
    }
  }
  return f;
}

} // namespace symbolic
} // namespace tc
