// Semantic analysis of a parsed TC function.
//
// Turns (apply ...) into (access ...) or (built-in ...), gives every expression a scalar type,
// discovers reduction variables (index variables that do not appear on the left-hand side) and
// enforces the language rules.  Behaviour, messages and the shape of the checked tree follow the
// reference (tc/lang/sema.h:129-163 type promotion, :230-240 reduction variables, :242-370
// expressions, :498-620 statements, :668-671 builtin shadowing) and are pinned by the golden
// dumps sema.expected, sema-env.expected, builtins.expected, indirect.expected, maxeq.expected
// and annotate.expected.
#pragma once
#include <algorithm>
#include <iostream>
#include <unordered_map>
#include <unordered_set>

#include "tc/lang/tree.h"
#include "tc/utils/compiler_options.h"

namespace lang {

// name -> arity of the math functions a TC may call (table of tc/lang/builtins.h:23-95)
inline const std::unordered_map<std::string, size_t>& builtinFunctions() {
  static const std::unordered_map<std::string, size_t> t = {
      {"acos", 1}, {"acosh", 1}, {"asin", 1}, {"asinh", 1}, {"atan2", 2}, {"atan", 1}, {"atanh", 1},
      {"cbrt", 1}, {"ceil", 1}, {"copysign", 2}, {"cos", 1}, {"cosh", 1}, {"cospi", 1},
      {"cyl_bessel_i0", 1}, {"cyl_bessel_i1", 1}, {"erfc", 1}, {"erfcinv", 1}, {"erfcx", 1},
      {"erf", 1}, {"erfinv", 1}, {"exp10", 1}, {"exp2", 1}, {"exp", 1}, {"expm1", 1}, {"fabs", 1},
      {"fdim", 2}, {"fdivide", 2}, {"floor", 1}, {"fma", 3}, {"fmax", 2}, {"fmin", 2}, {"fmod", 2},
      {"hypot", 2}, {"j0", 1}, {"j1", 1}, {"lgamma", 1}, {"log10", 1}, {"log1p", 1}, {"log2", 1},
      {"logb", 1}, {"log", 1}, {"nextafter", 2}, {"norm3d", 3}, {"norm4d", 4}, {"normcdf", 1},
      {"normcdfinv", 1}, {"pow", 2}, {"rcbrt", 1}, {"remainder", 2}, {"rhypot", 2}, {"rnorm3d", 3},
      {"rnorm4d", 4}, {"round", 1}, {"rsqrt", 1}, {"sin", 1}, {"sinh", 1}, {"sinpi", 1}, {"sqrt", 1},
      {"tan", 1}, {"tanh", 1}, {"tgamma", 1}, {"trunc", 1}, {"y0", 1}, {"y1", 1}};
  return t;
}

// Scalar type as (class, bits); bool is a 1-bit unsigned integer.
struct TypeInfo {
  enum Code { Int = 0, UInt = 1, Float = 2 };
  Code code;
  int bits;
  TypeInfo(Code c, int b) : code(c), bits(b) {}
  explicit TypeInfo(const TreeRef& scalarType) : code(Int), bits(32) {
    switch (scalarType->kind()) {
      case TK_BOOL: code = UInt; bits = 1; break;
      case TK_UINT8: code = UInt; bits = 8; break;
      case TK_UINT16: code = UInt; bits = 16; break;
      case TK_UINT32: code = UInt; bits = 32; break;
      case TK_UINT64: code = UInt; bits = 64; break;
      case TK_INT8: code = Int; bits = 8; break;
      case TK_INT16: code = Int; bits = 16; break;
      case TK_INT32: code = Int; bits = 32; break;
      case TK_INT64: code = Int; bits = 64; break;
      case TK_FLOAT16: code = Float; bits = 16; break;
      case TK_FLOAT32: case TK_FLOAT: code = Float; bits = 32; break;
      case TK_FLOAT64: case TK_DOUBLE: code = Float; bits = 64; break;
      default:
        throw errorAt(scalarType) << "Unhandled TC scalar type: " << kindToString(scalarType->kind());
    }
    // (The reference stops here for float16, "until we can make NVRTC include system headers",
    // tc/lang/sema.h:62-66: hipRTC knows _Float16 without any header, so the type is carried on.)
  }
  bool isFloat() const { return code == Float; }
  bool isUInt() const { return code == UInt; }
  bool operator==(const TypeInfo& o) const { return code == o.code && bits == o.bits; }
  int toScalarToken() const {
    if (code == Float) {
      return bits == 16 ? TK_FLOAT16 : bits == 32 ? TK_FLOAT : TK_DOUBLE;
    }
    if (code == UInt) {
      switch (bits) {
        case 1: return TK_BOOL;
        case 8: return TK_UINT8;
        case 16: return TK_UINT16;
        case 32: return TK_UINT32;
        default: return TK_UINT64;
      }
    }
    switch (bits) {
      case 8: return TK_INT8;
      case 16: return TK_INT16;
      case 32: return TK_INT32;
      default: return TK_INT64;
    }
  }
};

// Binary promotion: float beats integer, wider float beats narrower, uint+uint stays uint,
// any other integer mix becomes a signed integer of the wider width.
inline TreeRef matchTypes(const TreeRef& a, const TreeRef& b) {
  TypeInfo ta(a), tb(b);
  if (ta == tb) {
    return a;
  }
  if (!ta.isFloat() && tb.isFloat()) {
    return b;
  }
  if (ta.isFloat() && !tb.isFloat()) {
    return a;
  }
  if (ta.isFloat() && tb.isFloat()) {
    return ta.bits > tb.bits ? a : b;
  }
  if (ta.isUInt() && tb.isUInt()) {
    return ta.bits > tb.bits ? a : b;
  }
  return Tree::make(TypeInfo(TypeInfo::Int, std::max(ta.bits, tb.bits)).toScalarToken(), a->range());
}

inline void warn(const ErrorReport& e, const tc::CompilerOptions& opts) {
  if (opts.throwWarnings) {
    throw e;
  }
  if (opts.emitWarnings) {
    std::cerr << "WARNING: " << e.what();
  }
}

class Sema {
 public:
  explicit Sema(const tc::CompilerOptions& opts = tc::CompilerOptions()) : opts_(opts) {}

  // Scalar type tree ((float), (int32), ...) of a checked expression.
  TreeRef typeOfExpr(const TreeRef& e) const {
    auto it = types_.find(e.get());
    if (it == types_.end()) {
      throw errorAt(e) << "INTERNAL ERROR: expression has no type";
    }
    return it->second;
  }

  TreeRef checkFunction(const TreeRef& funcTree) {
    Def func(funcTree);
    TreeList params;
    for (const auto& p : func.params()) {
      params.push_back(checkParam(p));
    }
    for (const auto& r : func.returns()) {
      Param ret(r);
      if (!ret.typeIsInferred()) {
        annotated_[ret.ident().name()] = ret.type();
      }
      declared_.insert(ret.ident().name());
    }
    for (const auto& p : func.params()) {
      std::string n = Param(p).ident().name();
      declared_.insert(n);
      inputs_.insert(n);
    }
    TreeList stmts;
    for (const auto& s : func.statements()) {
      stmts.push_back(checkStmt(s));
    }
    for (const auto& r : func.returns()) {
      lookup(env_, Param(r).ident(), true);
    }
    return Tree::make(
        TK_DEF, func.range(),
        {func.name(), makeList(funcTree->tree(1)->range(), std::move(params)), funcTree->tree(2),
         makeList(funcTree->tree(3)->range(), std::move(stmts))});
  }

  // "name: type" lines sorted by name (sema-env.expected)
  std::string dumpEnv() const {
    std::vector<std::pair<std::string, TreeRef>> v(env_.begin(), env_.end());
    std::sort(v.begin(), v.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    std::stringstream ss;
    for (const auto& p : v) {
      ss << p.first << ": " << p.second;
    }
    return ss.str();
  }

 private:
  using Env = std::unordered_map<std::string, TreeRef>;

  TreeRef typed(TreeRef e, TreeRef type) {
    types_[e.get()] = std::move(type);
    keepAlive_.push_back(e);
    return e;
  }
  TreeRef scalar(int kind, const TreeRef& anchor) { return Tree::make(kind, anchor->range()); }

  void insert(Env& env, const Ident& id, TreeRef value, bool mustBeNew) {
    if (builtinFunctions().count(id.name())) {
      throw errorAt(id) << "'" << id.name() << "' is a built-in function and cannot be redefined";
    }
    bool added = env.emplace(id.name(), std::move(value)).second;
    if (mustBeNew && !added) {
      throw errorAt(id) << id.name() << " already defined";
    }
  }
  TreeRef lookup(Env& env, const Ident& id, bool required) {
    auto it = env.find(id.name());
    if (it == env.end()) {
      if (required) {
        throw errorAt(id) << "undefined variable " << id.name() << " used here.";
      }
      return nullptr;
    }
    return it->second;
  }
  TreeRef lookup(const Ident& id, bool required) {
    if (TreeRef v = lookup(indexEnv_, id, false)) {
      return v;
    }
    if (TreeRef v = lookup(letEnv_, id, false)) {
      return v;
    }
    return lookup(env_, id, required);
  }

  TreeRef checkParam(const TreeRef& p) {
    Param param(p);
    TensorType tt(param.type());
    for (const auto& d : tt.dims()) {
      if (d->kind() == TK_IDENT) {
        insert(env_, Ident(d), scalar(TK_INT32, d), false);
      }
    }
    insert(env_, param.ident(), param.type(), true);
    return p;
  }

  TreeRef matchAll(const TreeRef& list, TreeRef seed = nullptr) {
    for (const auto& e : list->trees()) {
      seed = seed ? matchTypes(seed, typeOfExpr(e)) : typeOfExpr(e);
    }
    return seed;
  }
  TreeRef expectIntegral(const TreeRef& e) {
    if (TypeInfo(typeOfExpr(e)).isFloat()) {
      throw errorAt(e) << " expected integral type but found " << kindToString(typeOfExpr(e)->kind());
    }
    return e;
  }
  void expectBool(const TreeRef& anchor, int kind) {
    if (kind != TK_BOOL) {
      throw errorAt(anchor) << "expected boolean but found " << kindToString(kind);
    }
  }

  TreeRef checkChildren(const TreeRef& e, bool allowAccess) {
    return e->map([&](TreeRef c) { return checkExp(c, allowAccess); });
  }

  TreeRef checkExp(const TreeRef& e, bool allowAccess) {
    switch (e->kind()) {
      case TK_APPLY: {
        if (!allowAccess) {
          throw errorAt(e) << "tensor accesses cannot be used in this context";
        }
        Apply a(e);
        Ident name = a.name();
        auto bi = builtinFunctions().find(name.name());
        if (bi != builtinFunctions().end()) {
          if (bi->second != a.arguments().size()) {
            throw errorAt(e) << "expected " << bi->second << " but found " << a.arguments().size();
          }
          TreeRef args = checkChildren(a.argumentList(), allowAccess);
          // math functions are float unless an argument is wider
          TreeRef type = matchAll(args, scalar(TK_FLOAT, e));
          return typed(BuiltIn::create(e->range(), name.name(), args, type), type);
        }
        TreeRef t = lookup(name, true);
        if (t->kind() != TK_TENSOR_TYPE) {
          throw errorAt(name) << "expected a tensor but found a scalar";
        }
        TensorType tt(t);
        if (tt.dims().size() != a.arguments().size()) {
          throw errorAt(e) << "expected " << tt.dims().size() << " dimensions but found "
                           << a.arguments().size() << " dimensions.";
        }
        TreeRef args = checkChildren(a.argumentList(), allowAccess);
        for (const auto& x : args->trees()) {
          expectIntegral(x);
        }
        return typed(Apply::create(TK_ACCESS, e->range(), name, args), tt.scalarTypeTree());
      }
      case TK_IDENT: {
        Ident id(e);
        TreeRef t = lookup(id, false);
        if (!t) { // unknown name: a new reduction index
          t = scalar(TK_INT32, e);
          insert(indexEnv_, id, t, true);
          reductionVars_.push_back(e);
        }
        if (t->kind() == TK_TENSOR_TYPE) {
          if (!TensorType(t).dims().empty()) {
            throw errorAt(e) << "expected a scalar but found a tensor expression.";
          }
          return checkExp(Apply::create(TK_APPLY, e->range(), e, makeList(e->range())), allowAccess);
        }
        return typed(e, t);
      }
      case '+': case '-': case '*': case '/': case '%': case TK_MIN: case TK_MAX: {
        TreeRef n = checkChildren(e, allowAccess);
        return typed(n, matchAll(n));
      }
      case TK_EQ: case TK_NE: case TK_GE: case TK_LE: case '<': case '>': {
        TreeRef n = checkChildren(e, allowAccess);
        matchAll(n);
        return typed(n, scalar(TK_BOOL, e));
      }
      case TK_AND: case TK_OR: case '!': {
        TreeRef n = checkChildren(e, allowAccess);
        expectBool(e, matchAll(n)->kind());
        return typed(n, scalar(TK_BOOL, e));
      }
      case '?': {
        TreeRef n = checkChildren(e, allowAccess);
        expectBool(n->tree(0), typeOfExpr(n->tree(0))->kind());
        return typed(n, matchTypes(typeOfExpr(n->tree(1)), typeOfExpr(n->tree(2))));
      }
      case TK_CONST:
        return typed(e, Const(e).type());
      case TK_CAST: {
        Cast c(e);
        TreeRef v = checkExp(c.value(), allowAccess);
        matchTypes(typeOfExpr(v), c.type());
        return typed(Tree::make(TK_CAST, e->range(), {v, c.type()}), c.type());
      }
      case TK_LIST:
        return checkChildren(e, allowAccess);
      default:
        throw errorAt(e) << "NYI - semantic checking for " << kindToString(e->kind());
    }
  }

  TreeRef checkWhereClause(const TreeRef& w) {
    if (w->kind() == TK_LET) {
      Let l(w);
      TreeRef rhs = checkExp(l.rhs(), true);
      insert(letEnv_, l.name(), typeOfExpr(rhs), true);
      return Tree::make(TK_LET, w->range(), {l.name(), rhs});
    }
    if (w->kind() == TK_EXISTS) {
      return Tree::make(TK_EXISTS, w->range(), {checkExp(w->tree(0), true)});
    }
    RangeConstraint rc(w);
    // a range may name an index the right-hand side has not introduced yet
    if (!lookup(rc.ident(), false)) {
      insert(indexEnv_, rc.ident(), scalar(TK_INT32, rc.ident()), true);
      reductionVars_.push_back(rc.ident());
    }
    lookup(indexEnv_, rc.ident(), true);
    TreeRef s = expectIntegral(checkExp(rc.start(), false));
    TreeRef e = expectIntegral(checkExp(rc.end(), false));
    return Tree::make(TK_RANGE_CONSTRAINT, w->range(), {rc.ident(), s, e});
  }

  static bool isPlainReduction(int k) {
    return k == TK_PLUS_EQ || k == TK_TIMES_EQ || k == TK_MIN_EQ || k == TK_MAX_EQ;
  }

  TreeRef checkStmt(const TreeRef& stmtTree) {
    Comprehension stmt(stmtTree);
    for (const auto& idx : stmt.indices()) {
      insert(indexEnv_, Ident(idx), scalar(TK_INT32, idx), true);
    }
    std::string name = stmt.ident().name();
    if (inputs_.count(name)) {
      throw errorAt(stmtTree) << "TC inputs are immutable";
    }
    TreeList outputDims;
    for (size_t i = 0; i < stmt.indices().size(); ++i) {
      outputDims.push_back(Ident::create(stmt.range(), name + "." + std::to_string(i)));
    }
    // where clauses first: their let bindings are visible on the right-hand side
    TreeRef where = stmtTree->tree(4)->map([&](TreeRef w) { return checkWhereClause(w); });
    TreeRef rhs = checkExp(stmt.rhs(), true);
    TreeRef scalarType = typeOfExpr(rhs);

    auto ann = annotated_.find(name);
    if (ann != annotated_.end()) {
      TensorType tt(ann->second);
      TreeRef m = matchTypes(scalarType, tt.scalarTypeTree());
      if (TypeInfo(tt.scalarTypeTree()).toScalarToken() != TypeInfo(m).toScalarToken()) {
        throw errorAt(stmtTree) << " attempting to assign type " << kindToString(scalarType->kind())
                                << " to narrower type " << kindToString(tt.scalarType())
                                << " without an explicit cast";
      }
      if (tt.dims().size() != stmt.indices().size()) {
        throw errorAt(stmtTree) << " tensor defined with " << stmt.indices().size()
                                << " dimensions but declared as an output with " << tt.dims().size()
                                << " dimensions.";
      }
    }
    // An earlier statement defined the tensor: this one must write it with as many subscripts.
    // (The reference's sema lets the mismatch through, tc/lang/sema.h:566-571, and Halide refuses
    // the update definition afterwards; here nothing behind sema would notice.)
    if (TreeRef earlier = lookup(env_, stmt.ident(), false)) {
      if (earlier->kind() == TK_TENSOR_TYPE && TensorType(earlier).dims().size() != stmt.indices().size()) {
        throw errorAt(stmtTree) << name << " was defined with " << TensorType(earlier).dims().size()
                                << " dimensions and is written here with " << stmt.indices().size();
      }
    }
    if (isPlainReduction(stmt.assignment()->kind()) && !lookup(stmt.ident(), false)) {
      ErrorReport w(stmtTree->range());
      std::string tk = kindToToken(stmt.assignment()->kind());
      w << "Reduction without initialization. If " << name
        << " is not pre-initialized before calling the TC function,"
        << " consider using the !-suffixed reduction operator " << tk << "! instead of " << tk;
      warn(w, opts_);
    }
    insert(env_, stmt.ident(),
           TensorType::create(stmt.range(), scalarType, makeList(stmt.range(), std::move(outputDims))),
           false);

    TreeRef equivalent = stmt.equivalent();
    if (!equivalent->trees().empty()) {
      TreeRef eq = equivalent->tree(0);
      TreeRef accesses = eq->tree(1)->map([&](TreeRef a) { return checkExp(a, true); });
      equivalent = Tree::make(
          TK_OPTION, equivalent->range(), {Tree::make(TK_EQUIVALENT, eq->range(), {eq->tree(0), accesses})});
    }
    if (!reductionVars_.empty() && stmt.assignment()->kind() == '=') {
      throw errorAt(stmtTree) << "this statement includes reduction variable '"
                              << Ident(reductionVars_.back()).name()
                              << "' but does not specify a reduction.";
    }
    TreeRef reductions = makeList(stmt.ident().range(), std::move(reductionVars_));
    reductionVars_.clear();
    if (!declared_.count(name)) {
      throw errorAt(stmtTree) << name
                              << " is not listed as an input or output to this function. Temporaries tensors are not yet implemented";
    }
    indexEnv_.clear();
    letEnv_.clear();
    return Tree::make(
        TK_COMPREHENSION, stmt.range(),
        {stmt.ident(), stmtTree->tree(1), stmt.assignment(), rhs, where, equivalent, reductions});
  }

  tc::CompilerOptions opts_;
  Env env_, indexEnv_, letEnv_, annotated_;
  std::unordered_set<std::string> inputs_, declared_;
  TreeList reductionVars_;
  std::unordered_map<const Tree*, TreeRef> types_;
  TreeList keepAlive_;
};

// Renames every identifier to i0, i1, ... in order of first appearance so that two TCs that
// differ only in names print identically (cache key; tc/lang/canonicalize.h:29-68).
inline TreeRef canonicalize(const TreeRef& checked) {
  std::unordered_map<std::string, std::string> names;
  std::function<TreeRef(TreeRef)> go = [&](TreeRef n) -> TreeRef {
    if (n->kind() == TK_IDENT) {
      const std::string& old = Ident(n).name();
      auto it = names.find(old);
      if (it == names.end()) {
        it = names.emplace(old, "i" + std::to_string(names.size())).first;
      }
      return Ident::create(n->range(), it->second);
    }
    if (n->kind() == TK_APPLY) {
      throw errorAt(n) << "canonicalize needs a tree that went through semantic analysis";
    }
    return n->map(go);
  };
  return go(checked);
}

} // namespace lang
