#include "tc/core/mapper/mapper.h"
#include "tc/core/mapper/sync_placement.h"

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <functional>
#include <set>
#include <sstream>

#include "tc/core/check.h"
#include "tc/core/hip/hip_libraries.h"

namespace tc {
namespace mapper {
namespace {

using ir::Affine;
using ir::Expr;
using ir::ExprRef;
using ir::ReduceOp;
using ir::ScalarType;

// ------------------------------------------------------------------------------------------
// expression helpers
// ------------------------------------------------------------------------------------------
ExprRef mkExpr(Expr::Kind k, ScalarType t, std::string name, std::vector<ExprRef> args) {
  auto e = std::make_shared<Expr>();
  e->kind = k;
  e->type = t;
  e->name = std::move(name);
  e->args = std::move(args);
  return e;
}
ExprRef mkInt(int64_t v) {
  auto e = std::make_shared<Expr>();
  e->kind = Expr::IntImm;
  e->type = ScalarType{ScalarType::Int, 32};
  e->ival = v;
  return e;
}
ExprRef mkVar(const std::string& n) {
  return mkExpr(Expr::Var, ScalarType{ScalarType::Int, 32}, n, {});
}
ExprRef mkBin(const std::string& op, ExprRef a, ExprRef b) {
  return mkExpr(Expr::Binary, ScalarType{ScalarType::Int, 32}, op, {std::move(a), std::move(b)});
}

// Rebuilds `e` bottom-up; `fn` may return a replacement for a node (after its children were
// rewritten) or nullptr to keep it.
ExprRef rewrite(const ExprRef& e, const std::function<ExprRef(const ExprRef&)>& fn) {
  std::vector<ExprRef> args;
  bool changed = false;
  for (const auto& a : e->args) {
    ExprRef n = rewrite(a, fn);
    changed |= n != a;
    args.push_back(n);
  }
  ExprRef cur = e;
  if (changed) {
    auto c = std::make_shared<Expr>(*e);
    c->args = std::move(args);
    cur = c;
  }
  ExprRef r = fn(cur);
  return r ? r : cur;
}

void visit(const ExprRef& e, const std::function<void(const ExprRef&)>& fn) {
  fn(e);
  for (const auto& a : e->args) {
    visit(a, fn);
  }
}

// Visits only what every evaluation of `e` evaluates: not the branches of a select and not the
// right-hand side of a short-circuit operator.  A load found this way may be issued ahead of the
// expression; one guarded by a condition may address outside its tensor when the guard is false.
void visitUnconditional(const ExprRef& e, const std::function<void(const ExprRef&)>& fn) {
  fn(e);
  size_t n = e->args.size();
  if (e->kind == Expr::Select) n = 1;
  if (e->kind == Expr::Binary && (e->name == "&&" || e->name == "||")) n = 1;
  for (size_t i = 0; i < n; ++i) {
    visitUnconditional(e->args[i], fn);
  }
}

bool sameExpr(const ExprRef& a, const ExprRef& b) {
  if (a->kind != b->kind || a->name != b->name || a->ival != b->ival || a->fval != b->fval ||
      a->args.size() != b->args.size() || a->type != b->type) {
    return false;
  }
  for (size_t i = 0; i < a->args.size(); ++i) {
    if (!sameExpr(a->args[i], b->args[i])) {
      return false;
    }
  }
  return true;
}

bool affineEqual(const Affine& a, const Affine& b) {
  return a.valid && b.valid && a.coef == b.coef && a.constant == b.constant;
}

ScalarType matchType(const ScalarType& a, const ScalarType& b) {
  if (a == b) return a;
  if (!a.isFloat() && b.isFloat()) return b;
  if (a.isFloat() && !b.isFloat()) return a;
  if (a.isFloat() && b.isFloat()) return a.bits > b.bits ? a : b;
  if (a.code == ScalarType::UInt && b.code == ScalarType::UInt) return a.bits > b.bits ? a : b;
  return ScalarType{ScalarType::Int, std::max(a.bits, b.bits)};
}

std::string floatLiteral(double v, const ScalarType& t) {
  char buf[64];
  std::snprintf(buf, sizeof(buf), t.bits == 64 ? "%.17g" : "%.9g", v);
  std::string s = buf;
  if (s.find_first_of(".en") == std::string::npos) {
    s += ".0";
  }
  if (s.find("inf") != std::string::npos || s.find("nan") != std::string::npos) {
    return v > 0 ? "(1.0f/0.0f)" : "(-1.0f/0.0f)";
  }
  return t.bits == 64 ? s : s + "f";
}

int64_t ceilDiv(int64_t a, int64_t b) {
  return (a + b - 1) / b;
}

const char* axisName(int a) {
  return a == 0 ? "x" : a == 1 ? "y" : "z";
}

// ------------------------------------------------------------------------------------------
// stage formation and kernel grouping
// ------------------------------------------------------------------------------------------
struct RawStage {
  std::vector<const ir::Statement*> stmts;
  const ir::Statement& first() const { return *stmts.front(); }
};

// subscripts of every access to `tensor` in the statement's right-hand side
std::vector<std::vector<ExprRef>> accessesTo(const ir::Statement& s, const std::string& tensor) {
  std::vector<std::vector<ExprRef>> out;
  visit(s.rhs, [&](const ExprRef& e) {
    if (e->kind == Expr::Load && e->name == tensor) {
      out.push_back(e->args);
    }
  });
  return out;
}

bool isIdentityAccess(const std::vector<ExprRef>& subs, const std::vector<std::string>& lhsVars) {
  if (subs.size() != lhsVars.size()) {
    return false;
  }
  for (size_t i = 0; i < subs.size(); ++i) {
    if (subs[i]->kind != Expr::Var || subs[i]->name != lhsVars[i]) {
      return false;
    }
  }
  return true;
}

bool sameBox(const ir::Statement& a, const ir::Statement& b) {
  if (a.tensor != b.tensor || a.lhsVars != b.lhsVars) {
    return false;
  }
  for (const auto& v : a.lhsVars) {
    const ir::Range &ra = a.ranges.at(v), &rb = b.ranges.at(v);
    if (ra.min != rb.min || ra.max != rb.max) {
      return false;
    }
  }
  return true;
}

std::set<std::string> tensorsRead(const ir::Statement& s) {
  std::set<std::string> r;
  visit(s.rhs, [&](const ExprRef& e) {
    if (e->kind == Expr::Load) {
      r.insert(e->name);
    }
  });
  if (s.op != ReduceOp::None && !s.init) {
    r.insert(s.tensor);
  }
  return r;
}

// Largest d such that the dependence between stages A (earlier) and B is point-wise in the
// first d left-hand-side positions of both, or -1 when they cannot share a kernel.
int sharedPrefix(const RawStage& A, const RawStage& B) {
  const ir::Statement &a0 = A.first(), &b0 = B.first();
  size_t d = std::min(a0.lhsVars.size(), b0.lhsVars.size());
  for (size_t p = 0; p < d; ++p) {
    const ir::Range &ra = a0.ranges.at(a0.lhsVars[p]), &rb = b0.ranges.at(b0.lhsVars[p]);
    if (ra.min != rb.min || ra.max != rb.max) {
      d = p;
      break;
    }
  }
  auto limitBy = [&](const RawStage& reader, const std::string& tensor, size_t tensorRank) {
    // every access of `reader` to `tensor` must use its own p-th index at position p
    for (const auto* s : reader.stmts) {
      for (const auto& subs : accessesTo(*s, tensor)) {
        size_t ok = 0;
        while (ok < d && ok < tensorRank && ok < subs.size() && subs[ok]->kind == Expr::Var &&
               subs[ok]->name == s->lhsVars[ok]) {
          ++ok;
        }
        d = std::min(d, ok);
      }
    }
  };
  // RAW / WAW: B touches what A wrote
  limitBy(B, a0.tensor, a0.lhsVars.size());
  if (a0.tensor == b0.tensor) {
    return -1; // same tensor, different box: keep apart
  }
  // WAR: A read what B writes
  limitBy(A, b0.tensor, b0.lhsVars.size());
  return static_cast<int>(d);
}

// ------------------------------------------------------------------------------------------
// stage canonicalisation: collapse + vector lanes
// ------------------------------------------------------------------------------------------
struct StageBuilder {
  const ir::Function& f;
  StagePlan st;

  explicit StageBuilder(const ir::Function& fn) : f(fn) {}

  LoopVar* var(const std::string& n) {
    for (auto& v : st.vars) {
      if (v.name == n) return &v;
    }
    return nullptr;
  }

  void init(const RawStage& raw) {
    const ir::Statement& s0 = raw.first();
    st.tensor = s0.tensor;
    for (const auto& v : s0.lhsVars) {
      st.lhsSubs.push_back(mkVar(v));
      LoopVar lv;
      lv.name = v;
      lv.min = s0.ranges.at(v).min;
      lv.extent = s0.ranges.at(v).extent();
      st.vars.push_back(lv);
    }
    st.numParallel = static_cast<int>(st.vars.size());
    int redId = 0;
    for (const auto* s : raw.stmts) {
      StageStmt ss;
      ss.op = s->op;
      ss.init = s->init;
      ss.type = s->type;
      ExprRef rhs = s->rhs;
      // reduction variables get stage-unique names (two statements may both use "k")
      for (const auto& r : s->redVars) {
        std::string nn = r;
        if (var(nn)) {
          nn = r + "_" + std::to_string(redId);
        }
        ++redId;
        if (nn != r) {
          rhs = rewrite(rhs, [&](const ExprRef& e) -> ExprRef {
            return (e->kind == Expr::Var && e->name == r) ? mkVar(nn) : nullptr;
          });
        }
        LoopVar lv;
        lv.name = nn;
        lv.min = s->ranges.at(r).min;
        lv.extent = s->ranges.at(r).extent();
        lv.reduction = true;
        st.vars.push_back(lv);
        ss.redVars.push_back(nn);
      }
      ss.rhs = rhs;
      st.stmts.push_back(ss);
    }
    auto addView = [&](const ir::Tensor& t, bool out) {
      TensorView v;
      v.name = t.name;
      v.type = t.type;
      v.extents = t.extents;
      v.isOutput = out;
      st.views[t.name] = v;
    };
    for (const auto& t : f.inputs) addView(t, false);
    for (const auto& t : f.outputs) addView(t, true);
  }

  // variables used as values or inside non-affine subscripts cannot be merged or split
  std::set<std::string> looseVars() {
    std::set<std::string> loose;
    std::function<void(const ExprRef&, bool)> walk = [&](const ExprRef& e, bool inAffineSub) {
      if (e->kind == Expr::Var && !inAffineSub) {
        loose.insert(e->name);
      }
      if (e->kind == Expr::Load) {
        for (const auto& a : e->args) {
          walk(a, ir::toAffine(a).valid);
        }
        return;
      }
      for (const auto& a : e->args) {
        walk(a, inAffineSub);
      }
    };
    for (const auto& s : st.stmts) {
      walk(s.rhs, false);
    }
    return loose;
  }

  // all accesses (tensor, subscripts) of the stage including the store
  void forEachAccess(const std::function<void(const std::string&, const std::vector<ExprRef>&)>& fn) {
    fn(st.tensor, st.lhsSubs);
    for (const auto& s : st.stmts) {
      visit(s.rhs, [&](const ExprRef& e) {
        if (e->kind == Expr::Load) fn(e->name, e->args);
      });
    }
  }

  static bool mentions(const ExprRef& e, const std::string& v) {
    bool m = false;
    visit(e, [&](const ExprRef& x) { m |= x->kind == Expr::Var && x->name == v; });
    return m;
  }
  static bool isExactly(const ExprRef& e, const std::string& v) {
    Affine a = ir::toAffine(e);
    return a.valid && a.constant == 0 && a.coef.size() == 1 && a.coefOf(v) == 1;
  }

  // Merge adjacent variables a,b (two parallel ones, or two consecutive reduction variables of
  // one statement) when every access that mentions them has `a` alone in some dimension j and `b`
  // alone in dimension j+1 spanning that whole dimension: the pair then walks memory exactly
  // like one variable of extent |a|*|b| over the merged dimension, in the same order.
  bool tryCollapse(size_t k) {
    LoopVar &a = st.vars[k], &b = st.vars[k + 1];
    if (a.min != 0 || b.min != 0 || a.reduction != b.reduction) return false;
    StageStmt* owner = nullptr;
    if (a.reduction) {
      for (auto& s : st.stmts) {
        for (size_t i = 0; i + 1 < s.redVars.size(); ++i) {
          if (s.redVars[i] == a.name && s.redVars[i + 1] == b.name) owner = &s;
        }
      }
      if (!owner) return false;
    }
    auto loose = looseVars();
    if (loose.count(a.name) || loose.count(b.name)) return false;
    std::map<std::string, std::set<size_t>> mergeAt; // tensor -> dims j to merge with j+1
    bool ok = true;
    forEachAccess([&](const std::string& t, const std::vector<ExprRef>& subs) {
      bool any = false;
      for (const auto& s : subs) any |= mentions(s, a.name) || mentions(s, b.name);
      if (!any) return;
      size_t found = subs.size();
      for (size_t j = 0; j + 1 < subs.size(); ++j) {
        if (isExactly(subs[j], a.name) && isExactly(subs[j + 1], b.name)) found = j;
      }
      if (found == subs.size() || st.views.at(t).extents[found + 1] != b.extent) {
        ok = false;
        return;
      }
      for (size_t j = 0; j < subs.size(); ++j) {
        if (j != found && j != found + 1 && (mentions(subs[j], a.name) || mentions(subs[j], b.name))) {
          ok = false;
        }
      }
      mergeAt[t].insert(found);
    });
    if (!ok) return false;
    for (const auto& m : mergeAt) {
      if (m.second.size() != 1) return false; // one merge position per tensor
    }
    std::string merged = a.name + "_" + b.name;
    int64_t eb = b.extent;
    auto rewriteSubs = [&](const std::string& t, const std::vector<ExprRef>& subs) {
      auto it = mergeAt.find(t);
      if (it == mergeAt.end()) return subs;
      size_t j = *it->second.begin();
      std::vector<ExprRef> out(subs.begin(), subs.begin() + j);
      if (isExactly(subs[j], a.name) && isExactly(subs[j + 1], b.name)) {
        out.push_back(mkVar(merged));
      } else {
        out.push_back(mkBin("+", mkBin("*", subs[j], mkInt(st.views.at(t).extents[j + 1])), subs[j + 1]));
      }
      out.insert(out.end(), subs.begin() + j + 2, subs.end());
      return out;
    };
    st.lhsSubs = rewriteSubs(st.tensor, st.lhsSubs);
    for (auto& s : st.stmts) {
      s.rhs = rewrite(s.rhs, [&](const ExprRef& e) -> ExprRef {
        if (e->kind != Expr::Load || !mergeAt.count(e->name)) return nullptr;
        auto c = std::make_shared<Expr>(*e);
        c->args = rewriteSubs(e->name, e->args);
        return c;
      });
    }
    for (const auto& m : mergeAt) {
      auto& ext = st.views.at(m.first).extents;
      size_t j = *m.second.begin();
      ext[j] *= ext[j + 1];
      ext.erase(ext.begin() + j + 1);
    }
    if (owner) {
      auto it = std::find(owner->redVars.begin(), owner->redVars.end(), a.name);
      *it = merged;
      owner->redVars.erase(it + 1);
    } else {
      st.numParallel -= 1;
    }
    a.name = merged;
    a.extent *= eb;
    st.vars.erase(st.vars.begin() + k + 1);
    return true;
  }

  // Variables before `first` are shared with the other stages of the kernel and keep their shape.
  void collapse(size_t first = 0) {
    for (size_t k = first; k + 1 < st.vars.size();) {
      if (!tryCollapse(k)) ++k;
    }
  }

  // x = xo * V + xv with xv the innermost, always unrolled lane variable
  bool splitLanes(const std::string& name, int64_t V) {
    LoopVar* v = var(name);
    if (!v || V <= 1 || v->min != 0 || v->extent % V != 0 || v->extent == V) return false;
    if (looseVars().count(name)) return false;
    std::string xo = name + "_o", xv = name + "_v";
    ExprRef repl = mkBin("+", mkBin("*", mkVar(xo), mkInt(V)), mkVar(xv));
    auto sub = [&](const ExprRef& e) -> ExprRef {
      return (e->kind == Expr::Var && e->name == name) ? repl : nullptr;
    };
    for (auto& s : st.lhsSubs) s = rewrite(s, sub);
    for (auto& s : st.stmts) {
      s.rhs = rewrite(s.rhs, sub);
      for (size_t i = 0; i < s.redVars.size(); ++i) {
        if (s.redVars[i] == name) {
          s.redVars[i] = xo;
          s.redVars.insert(s.redVars.begin() + i + 1, xv);
          break;
        }
      }
    }
    size_t idx = v - &st.vars[0];
    LoopVar lane = *v;
    lane.name = xv;
    lane.extent = V;
    lane.vectorLane = true;
    st.vars[idx].name = xo;
    st.vars[idx].extent /= V;
    st.vars.insert(st.vars.begin() + idx + 1, lane);
    if (!lane.reduction) st.numParallel += 1;
    return true;
  }
};

// Decides whether a stage is a dense fp32 contraction the matrix cores can take and assigns the
// variable roles.  Needs: first statement `out +=(!) A(...) * B(...)` with affine subscripts,
// float operands, at least one parallel variable private to each operand; later statements are
// point-wise epilogues.
bool classifyContraction(StagePlan& st) {
  if (st.stmts.empty()) return false;
  const StageStmt& s = st.stmts[0];
  if (s.redVars.empty() || s.op != ReduceOp::Plus) return false;
  for (size_t i = 1; i < st.stmts.size(); ++i) {
    if (!st.stmts[i].redVars.empty()) return false;
  }
  ScalarType f32{ScalarType::Float, 32};
  if (st.views.at(st.tensor).type != f32) return false;
  const ExprRef& e = s.rhs;
  if (e->kind != Expr::Binary || e->name != "*" || e->args[0]->kind != Expr::Load || e->args[1]->kind != Expr::Load) {
    return false;
  }
  for (const auto& l : e->args) {
    if (l->type != f32 || l->name == st.tensor) return false;
    for (const auto& a : l->args) {
      if (!ir::toAffine(a).valid) return false;
    }
  }
  auto mentions = [](const ExprRef& load, const std::string& v) {
    bool m = false;
    visit(load, [&](const ExprRef& x) { m |= x->kind == Expr::Var && x->name == v; });
    return m;
  };
  std::vector<std::string> onlyA, onlyB, batch, k;
  for (const auto& v : st.vars) {
    if (v.vectorLane) return false;
    bool a = mentions(e->args[0], v.name), b = mentions(e->args[1], v.name);
    if (v.reduction) {
      k.push_back(v.name);
    } else if (a && !b) {
      onlyA.push_back(v.name);
    } else if (b && !a) {
      onlyB.push_back(v.name);
    } else {
      batch.push_back(v.name);
    }
  }
  if (onlyA.empty() || onlyB.empty() || k.empty()) return false;
  st.mfma = true;
  st.mfmaM = onlyA;
  st.mfmaN = onlyB;
  st.mfmaBatch = batch;
  st.mfmaK = k;
  st.mfmaSwapOperands = false;
  // The 16 lanes of a row group hold 16 consecutive N positions of the output tile: put the
  // output's innermost (contiguous) index on the N side so that stores coalesce.
  std::string innermost;
  for (const auto& v : st.vars) {
    if (!v.reduction) innermost = v.name;
  }
  if (std::find(onlyA.begin(), onlyA.end(), innermost) != onlyA.end()) {
    std::swap(st.mfmaM, st.mfmaN);
    st.mfmaSwapOperands = true;
  }
  return true;
}

// ------------------------------------------------------------------------------------------
// code emission
// ------------------------------------------------------------------------------------------
class Emitter {
 public:
  std::ostringstream out;
  int indent = 0;
  void line(const std::string& s) { out << std::string(indent * 2, ' ') << s << "\n"; }
  void open(const std::string& s) {
    line(s.empty() ? "{" : s + " {");
    ++indent;
  }
  void close() {
    --indent;
    line("}");
  }
};

// tensors a stage loads from (its own running value included when it re-reads it)
std::set<std::string> tensorsRead(const StagePlan& st) {
  std::set<std::string> r;
  for (const auto& stmt : st.stmts) {
    visit(stmt.rhs, [&](const ExprRef& e) {
      if (e->kind == Expr::Load) r.insert(e->name);
    });
  }
  return r;
}

struct KernelCtx {
  const ir::Function& f;
  const HipMappingOptions& opts;
  KernelPlan& k;
  std::string idx = "int"; // index arithmetic type
  int64_t NT() const { return k.block[0] * k.block[1] * k.block[2]; }
};

class StageCodegen {
 public:
  StageCodegen(KernelCtx& kc, StagePlan& st, int stageIdx, Emitter& em)
      : kc_(kc), st_(st), stageIdx_(stageIdx), em_(em) {}

  // --- naming -------------------------------------------------------------------------------
  std::string iv(const LoopVar& v) const { return "i_" + v.name; }
  std::string tv(const LoopVar& v) const {
    auto it = tileOverride.find(v.name);
    if (it != tileOverride.end()) return it->second;
    return v.numTiles > 1 ? "t_" + v.name : "0";
  }
  // while emitting the loads of a prefetched tile: tile-index expression to use for a variable
  std::map<std::string, std::string> tileOverride;
  // LDS staging is driven by the kernel-level pipeline: stages only declare footprint origins
  bool suppressCopy = false;

  const LoopVar& var(const std::string& n) const {
    for (const auto& v : st_.vars) {
      if (v.name == n) return v;
    }
    TC_CHECK(false) << "unknown loop variable " << n;
    return st_.vars[0];
  }

  // affine over i_<var> values -> C
  std::string affineStr(const Affine& a) const {
    std::ostringstream ss;
    bool first = true;
    for (const auto& c : a.coef) {
      if (c.second == 0) continue;
      int64_t k = c.second;
      if (!first) ss << (k < 0 ? " - " : " + ");
      else if (k < 0) ss << "-";
      int64_t m = k < 0 ? -k : k;
      if (m != 1) ss << m << " * ";
      ss << "i_" << c.first;
      first = false;
    }
    if (first) {
      ss << a.constant;
    } else if (a.constant != 0) {
      ss << (a.constant < 0 ? " - " : " + ") << (a.constant < 0 ? -a.constant : a.constant);
    }
    return ss.str();
  }

  // --- expressions --------------------------------------------------------------------------
  std::string castTo(const ExprRef& e, const ScalarType& t, const std::string& accRef) {
    std::string s = expr(e, accRef);
    if (e->type == t || t.isBool()) return s;
    return "((" + t.cName() + ")(" + s + "))";
  }

  // flattened element offset as an affine form of the stage's variables (invalid when a
  // subscript is not affine)
  Affine flatAffine(const std::string& tensor, const std::vector<ExprRef>& subs) const {
    const TensorView& v = st_.views.at(tensor);
    auto strides = makeStridesFromSizes(v.extents);
    Affine total;
    total.valid = true;
    for (size_t j = 0; j < subs.size(); ++j) {
      Affine a = ir::toAffine(subs[j]);
      if (!a.valid) {
        total.valid = false;
        return total;
      }
      for (const auto& c : a.coef) total.coef[c.first] += c.second * strides[j];
      total.constant += a.constant * strides[j];
    }
    return total;
  }

  std::string flatIndex(const std::string& tensor, const std::vector<ExprRef>& subs, const std::string& accRef) {
    const TensorView& v = st_.views.at(tensor);
    auto strides = makeStridesFromSizes(v.extents);
    Affine total;
    total.valid = true;
    std::string extra;
    for (size_t j = 0; j < subs.size(); ++j) {
      Affine a = ir::toAffine(subs[j]);
      if (a.valid) {
        for (const auto& c : a.coef) total.coef[c.first] += c.second * strides[j];
        total.constant += a.constant * strides[j];
      } else {
        extra += " + " + std::to_string(strides[j]) + " * (" + kc_.idx + ")(" + expr(subs[j], accRef) + ")";
      }
    }
    return affineStr(total) + extra;
  }

  // Larger than what the L2 of one XCD keeps between uses.
  static constexpr int64_t kStreamingBytes = 4 << 20;

  int64_t viewBytes(const std::string& tensor) const {
    const TensorView& v = st_.views.at(tensor);
    int64_t n = (v.type.bits + 7) / 8;
    for (int64_t e : v.extents) n *= e;
    return n;
  }

  // An operand every element of which is needed by one thread only (all parallel variables that
  // are spread over blocks, threads or sequential tile loops occur in its subscripts) and that is
  // too large to stay in cache anyway: loads of it carry the non-temporal hint.
  bool streamedOnce(const std::string& tensor, const std::vector<ExprRef>& subs) const {
    if (viewBytes(tensor) < kStreamingBytes) return false;
    std::set<std::string> used;
    for (const auto& sub : subs) {
      Affine a = ir::toAffine(sub);
      if (!a.valid) return false;
      for (const auto& c : a.coef) {
        if (c.second != 0) used.insert(c.first);
      }
    }
    for (int i = 0; i < st_.numParallel; ++i) {
      const LoopVar& v = st_.vars[i];
      if (v.extent == 1 || used.count(v.name)) continue;
      if (v.numTiles == 1 && v.threadAxis < 0) continue; // repeated inside one thread only
      return false;
    }
    return true;
  }

  // The stage's result when nothing later in this kernel reads it back and it is too large to be
  // found in cache by a later kernel: stores of it carry the non-temporal hint.
  bool streamedStore() const {
    if (!kc_.opts.useReadOnlyCacheValue || viewBytes(st_.tensor) < kStreamingBytes) return false;
    for (size_t j = stageIdx_ + 1; j < kc_.k.stages.size(); ++j) {
      if (tensorsRead(kc_.k.stages[j]).count(st_.tensor)) return false;
    }
    return true;
  }

  std::string storeStmt(const std::string& cond, const std::string& value) {
    std::string target = "p" + st_.tensor + "[" + flatIndex(st_.tensor, st_.lhsSubs, "") + "]";
    if (streamedStore()) return "if (" + cond + ") __builtin_nontemporal_store(" + value + ", &" + target + ");";
    return "if (" + cond + ") " + target + " = " + value + ";";
  }

  std::string loadStr(const ExprRef& e, const std::string& accRef) {
    // the stage's own running value
    if (e->name == st_.tensor && !accRef.empty() && e->args.size() == st_.lhsSubs.size()) {
      bool same = true;
      for (size_t i = 0; i < e->args.size(); ++i) same &= sameExpr(e->args[i], st_.lhsSubs[i]);
      if (same) return accRef;
    }
    for (const auto& p : st_.promotions) {
      if (p.tensor == e->name && activePromotions_.count(p.tensor)) {
        return p.ldsName + "[" + ldsIndex(p, e->args) + "]";
      }
    }
    std::string global = "p" + e->name + "[" + flatIndex(e->name, e->args, accRef) + "]";
    {
      auto it = hoistedLoads_.find(global);
      if (it != hoistedLoads_.end()) return it->second;
    }
    if (inCachedReduction_) {
      auto it = regCaches.find(global);
      if (it != regCaches.end()) {
        return it->second.name + "[" + cacheSlot_ + "]";
      }
    }
    if (kc_.opts.useReadOnlyCacheValue && !st_.views.at(e->name).isOutput && streamedOnce(e->name, e->args)) {
      // streaming read of an input that is never written: keep it out of the way of cached data
      global = "__builtin_nontemporal_load(&" + global + ")";
    }
    return global;
  }

  std::string expr(const ExprRef& e, const std::string& accRef) {
    switch (e->kind) {
      case Expr::IntImm:
        return std::to_string(e->ival);
      case Expr::FloatImm:
        return floatLiteral(e->fval, e->type);
      case Expr::Var:
        return "i_" + e->name;
      case Expr::Load:
        return loadStr(e, accRef);
      case Expr::Cast:
        return "((" + e->type.cName() + ")(" + expr(e->args[0], accRef) + "))";
      case Expr::Unary:
        return "(" + e->name + expr(e->args[0], accRef) + ")";
      case Expr::Select:
        return "(" + expr(e->args[0], accRef) + " ? " + castTo(e->args[1], e->type, accRef) + " : " +
            castTo(e->args[2], e->type, accRef) + ")";
      case Expr::Call: {
        std::string s = e->name + "(";
        for (size_t i = 0; i < e->args.size(); ++i) {
          s += (i ? ", " : "") + castTo(e->args[i], e->type, accRef);
        }
        return s + ")";
      }
      case Expr::Binary: {
        ScalarType mt = matchType(e->args[0]->type, e->args[1]->type);
        if (e->name == "&&" || e->name == "||") {
          return "(" + expr(e->args[0], accRef) + " " + e->name + " " + expr(e->args[1], accRef) + ")";
        }
        std::string a = castTo(e->args[0], mt, accRef), b = castTo(e->args[1], mt, accRef);
        if (e->name == "min") return "__tc::tmin(" + a + ", " + b + ")";
        if (e->name == "max") return "__tc::tmax(" + a + ", " + b + ")";
        if (e->name == "/" && !mt.isFloat()) return "__tc::floordiv(" + a + ", " + b + ")";
        if (e->name == "%" && !mt.isFloat()) return "__tc::floormod(" + a + ", " + b + ")";
        if (e->name == "%") return std::string(mt.bits == 64 ? "fmod(" : "fmodf(") + a + ", " + b + ")";
        return "(" + a + " " + e->name + " " + b + ")";
      }
    }
    return "0";
  }

  static std::string combine(ReduceOp op, const std::string& a, const std::string& b) {
    switch (op) {
      case ReduceOp::Plus: return "(" + a + " + " + b + ")";
      case ReduceOp::Times: return "(" + a + " * " + b + ")";
      case ReduceOp::Min: return "__tc::tmin(" + a + ", " + b + ")";
      case ReduceOp::Max: return "__tc::tmax(" + a + ", " + b + ")";
      default: return b;
    }
  }
  static std::string opStruct(ReduceOp op, const ScalarType& t) {
    const char* n = op == ReduceOp::Plus ? "OpSum" : op == ReduceOp::Times ? "OpProd" : op == ReduceOp::Min ? "OpMin" : "OpMax";
    return std::string("__tc::") + n + "<" + t.cName() + ">";
  }

  // --- LDS ------------------------------------------------------------------------------------
  // lower corner of a promoted tensor's footprint in view dimension j, as C on tile indices
  struct Footprint {
    std::vector<Affine> coefs;          // subscript structure shared by all accesses
    std::vector<int64_t> minConst;      // smallest constant per dimension over the accesses
  };
  std::map<std::string, Footprint> footprints_;

  // span of a variable inside the region a promotion covers, and its low value as C
  int64_t spanOf(const LoopVar& v, bool insideReductionTiles) const {
    if (v.reduction && !insideReductionTiles) return v.extent;
    return v.tile;
  }
  std::string lowOf(const LoopVar& v, bool insideReductionTiles) const {
    if ((v.reduction && !insideReductionTiles) || v.numTiles == 1) return std::to_string(v.min);
    return "(" + std::to_string(v.min) + " + " + tv(v) + " * " + std::to_string(v.tile) + ")";
  }

  std::string footprintLow(const Promotion& p, size_t j) const {
    const Footprint& fp = footprints_.at(p.tensor);
    std::ostringstream ss;
    ss << fp.minConst[j];
    for (const auto& c : fp.coefs[j].coef) {
      const LoopVar& v = var(c.first);
      if (c.second > 0) {
        ss << " + " << c.second << " * " << lowOf(v, p.insideReductionTiles);
      } else {
        ss << " - " << -c.second << " * (" << lowOf(v, p.insideReductionTiles) << " + "
           << spanOf(v, p.insideReductionTiles) - 1 << ")";
      }
    }
    return ss.str();
  }

  std::string ldsIndex(const Promotion& p, const std::vector<ExprRef>& subs) {
    std::ostringstream ss;
    for (size_t j = 0; j < subs.size(); ++j) {
      if (j) ss << " + ";
      ss << "((" << affineStr(ir::toAffine(subs[j])) << ") - lo" << stageIdx_ << "_" << p.tensor << "_" << j << ")";
      if (p.ldsStrides[j] != 1) ss << " * " << p.ldsStrides[j];
    }
    if (subs.empty()) ss << "0";
    return ss.str();
  }

  // Decide which read-only operands of statement `s` to stage in LDS.
  // Matrix-core stages whose block tile holds a single 16-row group of the M side: the M-side
  // operand of a wavefront is the same for all of its output tiles, so each lane keeps its
  // elements (one per reduction step) in registers for the whole stage instead of re-reading them.
  static constexpr int64_t kMaxResidentSteps = 64;
  static constexpr int64_t kMfmaPad = 4;
  bool mfmaKeepsMOperandInRegisters() const {
    if (!st_.mfma) return false;
    int64_t MT = 1, BT = 1, KT = 1;
    for (const auto& n : st_.mfmaM) MT *= var(n).tile;
    for (const auto& n : st_.mfmaBatch) BT *= var(n).tile;
    for (const auto& n : st_.mfmaK) KT *= var(n).tile;
    for (const auto& n : st_.mfmaK) {
      if (var(n).numTiles > 1) return false;
    }
    return MT <= 16 && BT == 1 && ceilDiv(KT, 4) <= kMaxResidentSteps;
  }

  void planPromotions(const StageStmt& s, int64_t& ldsBudgetBytes) {
    if (!kc_.opts.useSharedMemoryValue || s.redVars.empty()) return;
    for (const auto& v : st_.vars) {
      if (!st_.mfma && !v.reduction && !v.unrolled && v.perThread > 1) return; // needs a full register tile
    }
    bool reductionTiled = false;
    for (const auto& r : s.redVars) reductionTiled |= var(r).numTiles > 1;
    bool inside = reductionTiled &&
        (!kc_.opts.hasSharedDepth || kc_.opts.sharedDepthValue > static_cast<uint32_t>(st_.numParallel));
    // iterations of the statement inside the promoted region
    std::set<std::string> stmtVars;
    for (int i = 0; i < st_.numParallel; ++i) stmtVars.insert(st_.vars[i].name);
    for (const auto& r : s.redVars) stmtVars.insert(r);
    double iterations = 1;
    for (const auto& n : stmtVars) iterations *= static_cast<double>(spanOf(var(n), inside));

    std::map<std::string, std::vector<std::vector<Affine>>> accesses;
    std::set<std::string> bad;
    visit(s.rhs, [&](const ExprRef& e) {
      if (e->kind != Expr::Load || e->name == st_.tensor) return;
      std::vector<Affine> subs;
      for (const auto& a : e->args) {
        Affine x = ir::toAffine(a);
        if (!x.valid) bad.insert(e->name);
        subs.push_back(x);
      }
      accesses[e->name].push_back(subs);
    });
    struct Cand {
      Promotion p;
      Footprint fp;
      int64_t bytes;
    };
    std::vector<Cand> cands;
    std::string residentOperand;
    if (mfmaKeepsMOperandInRegisters()) {
      residentOperand = s.rhs->args[st_.mfmaSwapOperands ? 1 : 0]->name; // read once per wavefront
    }
    for (const auto& acc : accesses) {
      if (bad.count(acc.first) || acc.first == residentOperand) continue;
      const TensorView& view = st_.views.at(acc.first);
      if (view.isOutput) continue; // may be written by another stage of this kernel
      const auto& ref = acc.second.front();
      // an operand every thread of the block reads at the same address goes through the scalar
      // data cache (s_load into SGPRs); staging it in LDS would only add traffic
      bool uniform = !st_.mfma; // on the matrix cores every operand element differs per lane
      for (const auto& sub : ref) {
        for (const auto& cv : sub.coef) uniform &= var(cv.first).threadAxis < 0 || cv.second == 0;
      }
      if (uniform) continue;
      bool sameShape = true;
      for (const auto& a : acc.second) {
        for (size_t j = 0; j < a.size(); ++j) sameShape &= a[j].coef == ref[j].coef;
      }
      if (!sameShape) continue;
      Cand c;
      c.p.tensor = acc.first;
      c.p.ldsName = "lds" + std::to_string(stageIdx_) + "_" + acc.first;
      c.p.insideReductionTiles = inside;
      c.fp.coefs = ref;
      int64_t elems = 1;
      for (size_t j = 0; j < ref.size(); ++j) {
        int64_t lo = ref[j].constant, hi = ref[j].constant;
        for (const auto& a : acc.second) {
          lo = std::min(lo, a[j].constant);
          hi = std::max(hi, a[j].constant);
        }
        int64_t ext = 1 + (hi - lo);
        for (const auto& cv : ref[j].coef) {
          ext += std::abs(cv.second) * (spanOf(var(cv.first), inside) - 1);
        }
        c.fp.minConst.push_back(lo);
        c.p.extents.push_back(ext);
        elems *= ext;
      }
      c.p.reuse = static_cast<int64_t>(iterations * acc.second.size() / static_cast<double>(elems));
      if (c.p.reuse < 2) continue;
      // pad the innermost extent to an odd size when lanes walk a slower dimension
      std::vector<int64_t> padded = c.p.extents;
      if (!padded.empty() && padded.back() > 1 && padded.back() % 2 == 0 && lanesWalkOuterDim(ref)) {
        padded.back() += 1;
      }
      // Matrix-core operands: the 16 lanes of a group walk the M- (or N-) side variable.  When that
      // variable is not in the last subscript, consecutive lanes are a whole row apart and a row
      // length that is a multiple of 8 elements piles them onto few LDS banks: four elements of
      // padding spread 16 rows over 8 banks groups while rows stay 16-byte aligned for the copies.
      if (st_.mfma && ref.size() >= 2 && padded.back() % 8 == 0 && kMfmaPad > 0) {
        bool isA = acc.first == s.rhs->args[st_.mfmaSwapOperands ? 1 : 0]->name;
        const auto& side = isA ? st_.mfmaM : st_.mfmaN;
        bool inLast = false, elsewhere = false;
        for (const auto& n : side) {
          inLast |= ref.back().coefOf(n) != 0;
          for (size_t j = 0; j + 1 < ref.size(); ++j) elsewhere |= ref[j].coefOf(n) != 0;
        }
        if (elsewhere && !inLast) padded.back() += kMfmaPad;
      }
      c.p.ldsStrides = makeStridesFromSizes(padded);
      c.p.elems = 1;
      for (auto e : padded) c.p.elems *= e;
      c.bytes = c.p.elems * view.type.bytes();
      cands.push_back(c);
    }
    // most reused first, name as tie-break for determinism
    std::sort(cands.begin(), cands.end(), [](const Cand& a, const Cand& b) {
      return a.p.reuse != b.p.reuse ? a.p.reuse > b.p.reuse : a.p.tensor < b.p.tensor;
    });
    for (auto& c : cands) {
      if (c.bytes <= ldsBudgetBytes) {
        ldsBudgetBytes -= c.bytes;
        footprints_[c.p.tensor] = c.fp;
        st_.promotions.push_back(c.p);
      }
    }
  }

  bool lanesWalkOuterDim(const std::vector<Affine>& subs) const {
    const LoopVar* x = nullptr;
    for (const auto& v : st_.vars) {
      if (v.threadAxis == 0) x = &v;
    }
    if (!x || subs.empty()) return false;
    if (subs.back().coefOf(x->name) != 0) return false;
    for (size_t j = 0; j + 1 < subs.size(); ++j) {
      if (subs[j].coefOf(x->name) != 0) return true;
    }
    return false;
  }

  void emitLdsDecls() {
    for (const auto& p : st_.promotions) {
      em_.line("__shared__ __attribute__((aligned(16))) " + st_.views.at(p.tensor).type.cName() + " " + p.ldsName +
               "[" + std::to_string(p.elems) + "];");
    }
  }

  std::string loPrefix(const Promotion& p) const { return "lo" + std::to_string(stageIdx_) + "_" + p.tensor + "_"; }

  void declareLows(const Promotion& p) {
    for (size_t j = 0; j < p.extents.size(); ++j) {
      em_.line("const int " + loPrefix(p) + std::to_string(j) + " = " + footprintLow(p, j) + ";");
    }
  }

  // --- global -> LDS copies --------------------------------------------------------------------
  // Copy dimensions: trailing dimensions the footprint covers completely (and that are not
  // padded in LDS) are contiguous in both memories and fold into their outer neighbour, which
  // removes most of the index decoding.  When the innermost copy dimension is contiguous on both
  // sides and every row starts on a multiple of four elements, threads move 16-byte vectors.
  struct CopyDim {
    int64_t extent, tensorExtent, gStride, lStride;
    std::string lo;
    int64_t loGcd; // every value of `lo` is a multiple of this (0: lo is always 0)
  };
  struct CopyPlan {
    std::vector<CopyDim> dims;
    int64_t count = 1;  // elements
    int vec = 1;        // elements per thread and iteration
    int64_t iters = 1;  // iterations per thread
    std::string elemType, regType;
  };

  static int64_t gcd(int64_t a, int64_t b) {
    a = std::abs(a);
    b = std::abs(b);
    while (b) {
      int64_t t = a % b;
      a = b;
      b = t;
    }
    return a;
  }

  // a divisor of every value footprintLow(p, j) can take
  int64_t footprintLowGcd(const Promotion& p, size_t j) const {
    const Footprint& fp = footprints_.at(p.tensor);
    int64_t g = std::abs(fp.minConst[j]);
    for (const auto& c : fp.coefs[j].coef) {
      const LoopVar& v = var(c.first);
      bool fixed = (v.reduction && !p.insideReductionTiles) || v.numTiles == 1;
      g = gcd(g, c.second * v.min);
      if (!fixed) g = gcd(g, c.second * v.tile);
      if (c.second < 0) g = gcd(g, c.second * (spanOf(v, p.insideReductionTiles) - 1));
    }
    return g;
  }

  CopyPlan copyPlan(const Promotion& p) const {
    const TensorView& view = st_.views.at(p.tensor);
    auto gStridesFull = makeStridesFromSizes(view.extents);
    CopyPlan plan;
    for (auto e : p.extents) plan.count *= e;
    for (size_t j = 0; j < p.extents.size(); ++j) {
      plan.dims.push_back(CopyDim{p.extents[j], view.extents[j], gStridesFull[j], p.ldsStrides[j],
                                  loPrefix(p) + std::to_string(j), footprintLowGcd(p, j)});
    }
    auto& dims = plan.dims;
    while (dims.size() >= 2) {
      CopyDim& in = dims.back();
      CopyDim& out = dims[dims.size() - 2];
      bool full = in.extent == in.tensorExtent && out.lStride == in.lStride * in.extent &&
          out.gStride == in.gStride * in.tensorExtent;
      if (!full) break;
      // (out, in) -> one dimension of extent out*in starting at out.lo * in.extent (in.lo is 0)
      out.lo = "(" + out.lo + ") * " + std::to_string(in.extent);
      out.loGcd *= in.extent;
      out.extent *= in.extent;
      out.tensorExtent *= in.tensorExtent;
      out.gStride = in.gStride;
      out.lStride = in.lStride;
      dims.pop_back();
    }
    plan.elemType = view.type.cName();
    plan.regType = plan.elemType;
    if (view.type.isFloat() && view.type.bits == 32 && !dims.empty()) {
      const CopyDim& in = dims.back();
      bool ok = in.gStride == 1 && in.lStride == 1 && in.extent % 4 == 0 && in.tensorExtent % 4 == 0 &&
          in.loGcd % 4 == 0;
      for (size_t j = 0; j + 1 < dims.size(); ++j) ok &= dims[j].gStride % 4 == 0 && dims[j].lStride % 4 == 0;
      if (ok) {
        plan.vec = 4;
        plan.regType = "__tc::floatx4";
      }
    }
    plan.iters = ceilDiv(plan.count / plan.vec, kc_.NT());
    return plan;
  }

  int64_t copyRegisters(const Promotion& p) const {
    CopyPlan plan = copyPlan(p);
    return plan.iters * plan.vec;
  }
  std::string copyRegisterDecl(const Promotion& p, const std::string& regs) const {
    CopyPlan plan = copyPlan(p);
    return plan.regType + " " + regs + "[" + std::to_string(plan.iters) + "];";
  }

  // One copy iteration of every thread: the global load of its element (vector) into
  // regs[slot], unconditional and from a clamped address so that loads issue back to back, or
  // the LDS store of regs[slot].
  void emitCopyStep(const Promotion& p, const CopyPlan& plan, const std::string& itExpr, const std::string& regs,
                    const std::string& slot, bool loads) {
    const auto& dims = plan.dims;
    std::string unit = "(" + itExpr + ") * " + std::to_string(kc_.NT()) + " + tid_";
    em_.line("const int c_ = " + (plan.vec > 1 ? std::to_string(plan.vec) + " * (" + unit + ")" : unit) + ";");
    int64_t div = plan.count;
    std::string cond = "c_ < " + std::to_string(plan.count), gidx, lidx;
    for (size_t j = 0; j < dims.size(); ++j) {
      div /= dims[j].extent;
      std::string l = "l" + std::to_string(j) + "_";
      std::string e = "c_";
      if (div > 1) e = "(" + e + " / " + std::to_string(div) + ")";
      if (j > 0) e = e + " % " + std::to_string(dims[j].extent);
      em_.line("const int " + l + " = " + e + ";");
      if (loads) {
        std::string g = "g" + std::to_string(j) + "_";
        em_.line("const int " + g + " = " + dims[j].lo + " + " + l + ";");
        cond += " && (unsigned)" + g + " < " + std::to_string(dims[j].tensorExtent) + "u";
        gidx += (j ? " + " : "") + g + (dims[j].gStride != 1 ? " * " + std::to_string(dims[j].gStride) : "");
      }
      lidx += (j ? " + " : "") + l + (dims[j].lStride != 1 ? " * " + std::to_string(dims[j].lStride) : "");
    }
    if (dims.empty()) gidx = lidx = "0";
    std::string cast = plan.vec > 1 ? "*(const __tc::floatx4u*)&" : "";
    std::string lcast = plan.vec > 1 ? "*(__tc::floatx4*)&" : "";
    if (loads) {
      em_.line(regs + "[" + slot + "] = " + cast + "p" + p.tensor + "[(" + cond + ") ? (" + gidx + ") : 0];");
    } else {
      em_.line("if (c_ < " + std::to_string(plan.count) + ") " + lcast + p.ldsName + "[" + lidx + "] = " + regs + "[" + slot + "];");
    }
  }

  // Whole-footprint variants used by the software pipeline: every thread keeps its share of the
  // tile in `regs` between the load and the store phase.  Footprint origins must be in scope.
  void emitCopyLoads(const Promotion& p, const std::string& regs) { emitCopyPhase(p, regs, true); }
  void emitCopyStores(const Promotion& p, const std::string& regs) { emitCopyPhase(p, regs, false); }

  void emitCopyPhase(const Promotion& p, const std::string& regs, bool loads) {
    CopyPlan plan = copyPlan(p);
    em_.line("#pragma unroll");
    em_.open("for (int it_ = 0; it_ < " + std::to_string(plan.iters) + "; ++it_)");
    emitCopyStep(p, plan, "it_", regs, "it_", loads);
    em_.close();
  }

  void emitCopyIn(const Promotion& p) {
    declareLows(p);
    CopyPlan plan = copyPlan(p);
    // Two phases per chunk of iterations: all global loads first, so that their latencies
    // overlap, then the LDS stores.
    int64_t chunk = std::min<int64_t>(plan.iters, (kc_.opts.unrollCopySharedValue ? 32 : 16) / plan.vec);
    chunk = std::max<int64_t>(chunk, 1);
    bool chunked = plan.iters > chunk;
    if (chunked) {
      em_.open("for (int cb_ = 0; cb_ < " + std::to_string(plan.iters) + "; cb_ += " + std::to_string(chunk) + ")");
    } else {
      em_.open("");
    }
    std::string base = chunked ? "cb_ + " : "";
    em_.line(plan.regType + " stage_[" + std::to_string(chunk) + "];");
    for (bool loads : {true, false}) {
      em_.line("#pragma unroll");
      em_.open("for (int it_ = 0; it_ < " + std::to_string(chunk) + "; ++it_)");
      emitCopyStep(p, plan, base + "it_", "stage_", "it_", loads);
      em_.close();
    }
    em_.close();
  }

  // --- loops ----------------------------------------------------------------------------------
  // Opens the per-thread point loop of `v` (uniform trip count across the block), declares
  // i_<v> and returns the predicate term this variable contributes ("" when always valid).
  std::string openPointLoop(const LoopVar& v, bool unrollPragma, int unrollFactor = 0) {
    std::string q = "q_" + v.name;
    std::string B = v.threadAxis >= 0 ? std::to_string(kc_.k.block[v.threadAxis]) : "1";
    if (v.perThread > 1) {
      if (unrollPragma) em_.line(unrollFactor > 1 ? "#pragma unroll " + std::to_string(unrollFactor) : "#pragma unroll");
      em_.open("for (int " + q + " = 0; " + q + " < " + std::to_string(v.perThread) + "; ++" + q + ")");
    } else {
      em_.open("");
    }
    std::string qv = v.perThread > 1 ? q : "0";
    std::string p;
    if (v.threadAxis >= 0) {
      p = qv == "0" ? std::string("(int)threadIdx.") + axisName(v.threadAxis)
                    : "(" + qv + " * " + B + " + (int)threadIdx." + axisName(v.threadAxis) + ")";
    } else {
      p = qv;
    }
    std::string base = std::to_string(v.min);
    if (v.numTiles > 1) base += " + " + tv(v) + " * " + std::to_string(v.tile);
    // Points outside the tile or the variable's range are folded onto the last valid point: the
    // folded iteration repeats valid work with in-bounds accesses, so loads and arithmetic need
    // no guard (straight-line code the compiler can vectorise and schedule freely); only the
    // stores and the reduction updates look at the predicate, which is taken before folding.
    bool overCover = v.threadAxis >= 0 && v.perThread * kc_.k.block[v.threadAxis] != v.tile;
    std::string pred;
    if (overCover) {
      em_.line("const int u_" + v.name + " = " + p + ";");
      em_.line("const int p_" + v.name + " = __tc::tmin(u_" + v.name + ", " + std::to_string(v.tile - 1) + ");");
      pred = "u_" + v.name + " < " + std::to_string(v.tile);
    } else {
      em_.line("const int p_" + v.name + " = " + p + ";");
    }
    if (v.partial()) {
      std::string last = std::to_string(v.min + v.extent - 1);
      em_.line("const int w_" + v.name + " = " + base + " + " + (overCover ? "u_" : "p_") + v.name + ";");
      em_.line("const int " + iv(v) + " = __tc::tmin(" + base + " + p_" + v.name + ", " + last + ");");
      pred += (pred.empty() ? "" : " && ") + std::string("w_") + v.name + " <= " + last;
    } else {
      em_.line("const int " + iv(v) + " = " + base + " + p_" + v.name + ";");
    }
    return pred;
  }

  // Register-tile loops: opens loops over all unrolled parallel variables, defines `ok_` and
  // the accumulator slot `a_`; the caller emits the body and then calls closeUnrolled().
  int openUnrolled() {
    em_.open("");
    int opened = 1;
    std::string pred = outerPred_;
    std::string slot = "0";
    for (int i = 0; i < st_.numParallel; ++i) {
      const LoopVar& v = st_.vars[i];
      if (!v.unrolled) continue;
      std::string t = openPointLoop(v, true);
      ++opened;
      if (!t.empty()) pred += (pred.empty() ? "" : " && ") + t;
      if (v.perThread > 1) slot = "(" + slot + ") * " + std::to_string(v.perThread) + " + q_" + v.name;
    }
    em_.line("const bool ok_ = " + (pred.empty() ? std::string("true") : pred) + ";");
    em_.line("const int a_ = " + slot + ";");
    return opened;
  }
  void closeN(int n) {
    for (int i = 0; i < n; ++i) em_.close();
  }

  // thread axes this stage does not use must not duplicate its work
  std::string idleAxesPred() const {
    std::string p;
    for (int a = 0; a < 3; ++a) {
      if (kc_.k.block[a] == 1) continue;
      bool used = false;
      for (const auto& v : st_.vars) used |= v.threadAxis == a;
      if (!used) p += (p.empty() ? "" : " && ") + std::string("threadIdx.") + axisName(a) + " == 0";
    }
    return p;
  }

  // --- statements -----------------------------------------------------------------------------
  void emitPointwise(const StageStmt& s) {
    int n = openUnrolled();
    inCachedReduction_ = cachedPointwise_;
    cacheSlot_ = "a_";
    em_.line("acc_[a_] = " + castTo(s.rhs, accType_, accValid_ ? "acc_[a_]" : "") + ";");
    inCachedReduction_ = false;
    closeN(n);
  }

  void preloadAcc() {
    int n = openUnrolled();
    em_.line("acc_[a_] = p" + st_.tensor + "[" + flatIndex(st_.tensor, st_.lhsSubs, "") + "];");
    closeN(n);
    accValid_ = true;
  }

  static bool readsOwnValue(const StageStmt& s, const StagePlan& st) {
    bool r = false;
    visit(s.rhs, [&](const ExprRef& e) { r |= e->kind == Expr::Load && e->name == st.tensor; });
    return r;
  }

  void emitReduction(const StageStmt& s, int64_t unrollBudget) {
    bool threadRed = false;
    for (const auto& r : s.redVars) threadRed |= st_.threadReduction && var(r).threadAxis == 0;
    std::string target = threadRed ? "part_" : "acc_";
    std::string ident = ir::identityLiteral(s.op, accType_);
    if (!s.init && !accValid_) preloadAcc();
    {
      int n = openUnrolled();
      if (threadRed) {
        em_.line("part_[a_] = " + ident + ";");
        if (s.init) em_.line("acc_[a_] = " + ident + ";");
      } else if (s.init) {
        em_.line("acc_[a_] = " + ident + ";");
      }
      closeN(n);
    }
    accValid_ = true;
    // promotions that cover the whole reduction go in front of the reduction loops
    bool anyOutside = false, anyInside = false;
    for (const auto& p : st_.promotions) (p.insideReductionTiles ? anyInside : anyOutside) = true;
    auto copyIn = [&](bool inside) {
      if (suppressCopy && !inside) {
        for (const auto& p : st_.promotions) {
          if (!p.insideReductionTiles) {
            declareLows(p);
            activePromotions_.insert(p.tensor);
          }
        }
        return;
      }
      em_.line("__syncthreads();");
      for (const auto& p : st_.promotions) {
        if (p.insideReductionTiles == inside) {
          emitCopyIn(p);
          activePromotions_.insert(p.tensor);
        }
      }
      em_.line("__syncthreads();");
    };
    int opened = 0;
    if (anyOutside) {
      em_.open("");
      ++opened;
      copyIn(false);
    }
    for (const auto& r : s.redVars) {
      const LoopVar& v = var(r);
      if (v.numTiles > 1) {
        em_.open("for (int t_" + v.name + " = 0; t_" + v.name + " < " + std::to_string(v.numTiles) + "; ++t_" + v.name + ")");
        ++opened;
      }
    }
    if (anyInside) copyIn(true);
    // point loops, innermost ones unrolled under the budget
    std::vector<int> factors(s.redVars.size(), 0); // 0: no pragma, -1: full, >1: partial
    int64_t remaining = std::max<int64_t>(1, unrollBudget / std::max<int64_t>(1, st_.accCount));
    bool cached = !regCaches.empty() && &s == cachedStmt_;
    if (cached) remaining = 1 << 30; // register-cached operands need fully unrolled loops
    for (int i = static_cast<int>(s.redVars.size()) - 1; i >= 0; --i) {
      const LoopVar& v = var(s.redVars[i]);
      if (v.vectorLane) {
        factors[i] = -1;
        continue;
      }
      if (v.perThread <= remaining) {
        factors[i] = -1;
        remaining /= std::max<int64_t>(1, v.perThread);
      } else {
        if (remaining >= 2) factors[i] = static_cast<int>(remaining);
        break;
      }
    }
    std::string rpred;
    int ropened = 0;
    for (size_t i = 0; i < s.redVars.size(); ++i) {
      const LoopVar& v = var(s.redVars[i]);
      std::string t = openPointLoop(v, factors[i] != 0, factors[i] > 1 ? factors[i] : 0);
      ++ropened;
      if (!t.empty()) rpred += (rpred.empty() ? "" : " && ") + t;
    }
    {
      int n = openUnrolled();
      // folded parallel points only repeat valid work and are never stored: the update is
      // guarded by the reduction's own predicate alone
      const std::string& cond = rpred;
      if (cached) {
        // slot of this (register-tile element, reduction iteration) in the per-thread cache
        std::string rlin = "0";
        int64_t rcount = 1;
        for (const auto& r : s.redVars) {
          const LoopVar& v = var(r);
          rcount *= v.perThread;
          if (v.perThread > 1) rlin = "(" + rlin + ") * " + std::to_string(v.perThread) + " + q_" + v.name;
        }
        cacheSlot_ = "a_ * " + std::to_string(rcount) + " + " + rlin;
        for (const auto& c : regCaches) {
          if (c.second.producer) {
            // the only read of the element from memory: streamed when the operand is large
            std::string tensor = c.first.substr(1, c.first.find('[') - 1);
            bool stream = kc_.opts.useReadOnlyCacheValue && !st_.views.at(tensor).isOutput &&
                viewBytes(tensor) >= kStreamingBytes;
            em_.line(c.second.name + "[" + cacheSlot_ + "] = " +
                     (stream ? "__builtin_nontemporal_load(&" + c.first + ")" : c.first) + ";");
          }
        }
        inCachedReduction_ = true;
      }
      std::string rhs = castTo(s.rhs, accType_, "acc_[a_]");
      inCachedReduction_ = false;
      if (cond.empty()) {
        em_.line(target + "[a_] = " + combine(s.op, target + "[a_]", rhs) + ";");
      } else {
        em_.line("const " + accType_.cName() + " r_ = " + rhs + ";");
        em_.line("if (" + cond + ") " + target + "[a_] = " + combine(s.op, target + "[a_]", "r_") + ";");
      }
      closeN(n);
    }
    closeN(ropened);
    closeN(opened);
    for (const auto& p : st_.promotions) activePromotions_.erase(p.tensor);
    if (threadRed) {
      // every thread of the block reaches this point (uniform loops), as the barriers require
      int n = openUnrolled();
      em_.line("const " + accType_.cName() + " tot_ = __tc::blockAllReduceX<" + opStruct(s.op, accType_) + ", " +
               std::to_string(kc_.k.block[0]) + ", " + std::to_string(kc_.k.block[1]) + ", " +
               std::to_string(kc_.k.block[2]) + ">(part_[a_], red_scratch_);");
      em_.line("acc_[a_] = " + combine(s.op, "acc_[a_]", "tot_") + ";");
      closeN(n);
    }
  }

  const std::vector<Promotion>& promotions() const { return st_.promotions; }
  std::string promotionType(const Promotion& p) const { return st_.views.at(p.tensor).type.cName(); }

  // --- register caches shared between stages -----------------------------------------------------
  struct RegCache {
    std::string name;
    bool producer = false;
  };
  std::map<std::string, RegCache> regCaches; // printed global load -> cache
  const StageStmt* cachedStmt_ = nullptr;

  const StageStmt* firstReduction() const {
    for (const auto& s : st_.stmts) {
      if (!s.redVars.empty()) return &s;
    }
    return nullptr;
  }

  // Loop structure + addressing of the stage's reduction statement in position-independent
  // form: two stages with equal signatures make every thread touch the same addresses at the
  // same loop counters.  Empty when the stage cannot take part in register caching.
  std::string cacheSignature(std::vector<std::pair<std::string, std::string>>& loads) {
    const StageStmt* s = firstReduction();
    if (!s) return "";
    std::map<std::string, std::string> canon;
    std::ostringstream sig;
    for (size_t i = 0; i < st_.vars.size(); ++i) {
      const LoopVar& v = st_.vars[i];
      bool mine = !v.reduction || std::find(s->redVars.begin(), s->redVars.end(), v.name) != s->redVars.end();
      if (!mine) return "";
      if (v.reduction && v.numTiles != 1) return "";
      if (!v.reduction && !v.unrolled && v.perThread > 1) return "";
      // the cache holds one tile: a tile loop that each stage runs by itself would reuse the
      // elements of its last iteration; loops opened around all stages are fine
      if (!v.reduction && !v.vectorLane && v.numTiles != 1 && static_cast<int>(i) >= kc_.k.sharedDepth &&
          !(v.blockAxis >= 0 && v.gridExtent == v.numTiles)) {
        return "";
      }
      canon[v.name] = "v" + std::to_string(i);
      sig << v.min << "," << v.extent << "," << v.tile << "," << v.numTiles << "," << v.blockAxis << ","
          << v.threadAxis << "," << v.perThread << "," << v.unrolled << "," << v.vectorLane << "," << v.reduction << ";";
    }
    visitUnconditional(s->rhs, [&](const ExprRef& e) {
      if (e->kind != Expr::Load) return;
      const TensorView& view = st_.views.at(e->name);
      if (view.isOutput) return;
      for (const auto& a : e->args) {
        if (!ir::toAffine(a).valid) return;
      }
      std::string text = "p" + e->name + "[" + flatIndex(e->name, e->args, "") + "]";
      // position-independent spelling of the same address
      std::string key = text;
      for (const auto& c : canon) {
        std::string from = "i_" + c.first, to = "#" + c.second;
        for (size_t pos = key.find(from); pos != std::string::npos; pos = key.find(from, pos + to.size())) {
          size_t end = pos + from.size();
          bool boundary = end >= key.size() || !(std::isalnum(static_cast<unsigned char>(key[end])) || key[end] == '_');
          if (boundary) key.replace(pos, from.size(), to);
        }
      }
      loads.emplace_back(key, text);
    });
    return sig.str();
  }

  int64_t cacheSlots() const {
    const StageStmt* s = firstReduction();
    int64_t n = st_.accCount;
    for (const auto& r : s->redVars) n *= var(r).perThread;
    return n;
  }

  // A load's flat element offset as a function of what tells threads and iterations apart: block
  // ids / kernel-level tile loops, thread ids, and the fully unrolled per-thread loop counters
  // named by their stride in the register-cache slot.  Two stages whose forms of an operand agree
  // make every thread touch the same element at the same slot, whatever their loop structure
  // (a reduction over one merged variable and a pointwise stage over (d, h*w), say).  Invalid
  // when a variable involved is clamped, folded, tiled inside the stage or loops without being
  // unrolled: the slot would then not name one element.
  struct AddressForm {
    bool valid = false;
    std::string tensor;
    int64_t constant = 0;
    int64_t slots = 1;
    std::map<std::string, int64_t> coef;
    bool operator==(const AddressForm& o) const {
      return valid && o.valid && tensor == o.tensor && constant == o.constant && slots == o.slots && coef == o.coef;
    }
  };
  AddressForm addressForm(const ExprRef& load, const StageStmt* reduction) const {
    AddressForm form;
    const TensorView& view = st_.views.at(load->name);
    if (view.isOutput) return form;
    Affine flat = flatAffine(load->name, load->args);
    if (!flat.valid) return form;
    // slot layout: unrolled parallel variables, then the statement's reduction variables
    std::vector<const LoopVar*> slotVars;
    for (int i = 0; i < st_.numParallel; ++i) {
      const LoopVar& v = st_.vars[i];
      if (v.perThread > 1 && !v.unrolled) return form;
      if (v.perThread > 1) slotVars.push_back(&v);
    }
    if (reduction) {
      for (const auto& r : reduction->redVars) {
        if (var(r).perThread > 1) slotVars.push_back(&var(r));
      }
    }
    std::map<std::string, int64_t> stride;
    for (size_t i = slotVars.size(); i-- > 0;) {
      stride[slotVars[i]->name] = form.slots;
      form.slots *= slotVars[i]->perThread;
    }
    for (const auto* sv : slotVars) {
      if (flat.coefOf(sv->name) == 0) return form; // a slot that does not move the address
    }
    form.tensor = load->name;
    form.constant = flat.constant;
    for (size_t i = 0; i < st_.vars.size(); ++i) {
      const LoopVar& v = st_.vars[i];
      int64_t c = flat.coefOf(v.name);
      if (c == 0) continue;
      bool mine = !v.reduction ||
          (reduction && std::find(reduction->redVars.begin(), reduction->redVars.end(), v.name) != reduction->redVars.end());
      if (!mine) return form;
      if (v.numTiles > 1 && (v.reduction || static_cast<int>(i) >= kc_.k.sharedDepth)) return form;
      bool blockId = v.blockAxis >= 0 && v.gridExtent == v.numTiles;
      std::string tileSym = blockId ? std::string("block.") + axisName(v.blockAxis) : "t_" + v.name;
      int64_t B = v.threadAxis >= 0 ? kc_.k.block[v.threadAxis] : 1;
      bool folded = v.partial() || (v.threadAxis >= 0 && v.perThread * B != v.tile);
      if (folded) {
        // the index is a clamped function of the same symbols: comparable only as a whole, between
        // variables that are tiled, spread and clamped alike
        std::ostringstream d;
        d << "folded(" << v.min << "," << v.extent << "," << v.tile << "," << v.numTiles << ","
          << (v.numTiles > 1 ? tileSym : std::string("-")) << "," << v.threadAxis << "," << B << "," << v.perThread << ","
          << (v.perThread > 1 ? stride.at(v.name) : 0) << ")";
        form.coef[d.str()] += c;
        continue;
      }
      form.constant += c * v.min;
      if (v.numTiles > 1) form.coef[tileSym] += c * v.tile;
      if (v.threadAxis >= 0) form.coef[std::string("thread.") + axisName(v.threadAxis)] += c;
      if (v.perThread > 1) form.coef["q." + std::to_string(stride.at(v.name))] += c * B;
    }
    form.valid = true;
    return form;
  }

  // Pointwise statements of this stage read the operands in `regCaches` from the register cache.
  bool cachedPointwise_ = false;

  // True when this stage touches `producer`'s result only at the element the same thread wrote:
  // both stages spread identical parallel variables over blocks and threads in the same way and
  // every access to the tensor uses the producer's own left-hand-side subscripts.
  bool readsPrivatelyFrom(const StagePlan& producer) const {
    if (producer.threadReduction || producer.mfma || st_.mfma) return false;
    if (producer.numParallel != st_.numParallel || producer.tensor == st_.tensor) return false;
    if (tensorsRead(producer).count(st_.tensor)) return false; // it also reads what this stage overwrites
    std::map<std::string, std::string> rename; // this stage's variable -> producer's
    for (int i = 0; i < st_.numParallel; ++i) {
      const LoopVar& a = producer.vars[i];
      const LoopVar& b = st_.vars[i];
      bool same = a.min == b.min && a.extent == b.extent && a.tile == b.tile && a.numTiles == b.numTiles &&
          a.blockAxis == b.blockAxis && a.gridExtent == b.gridExtent && a.threadAxis == b.threadAxis &&
          a.perThread == b.perThread && a.vectorLane == b.vectorLane;
      if (!same) return false;
      rename[b.name] = a.name;
    }
    if (producer.views.at(producer.tensor).extents != st_.views.at(producer.tensor).extents) return false;
    std::vector<Affine> lhs;
    for (const auto& e : producer.lhsSubs) lhs.push_back(ir::toAffine(e));
    bool ok = true;
    for (const auto& stmt : st_.stmts) {
      visit(stmt.rhs, [&](const ExprRef& e) {
        if (e->kind != Expr::Load || e->name != producer.tensor) return;
        ok = ok && e->args.size() == lhs.size();
        for (size_t j = 0; ok && j < lhs.size(); ++j) {
          Affine x = ir::toAffine(e->args[j]);
          ok = ok && x.valid && lhs[j].valid && x.constant == lhs[j].constant;
          std::map<std::string, int64_t> renamed;
          for (const auto& c : x.coef) {
            if (c.second == 0) continue;
            auto it = rename.find(c.first);
            if (it == rename.end()) {
              ok = false;
              break;
            }
            renamed[it->second] += c.second;
          }
          std::map<std::string, int64_t> want;
          for (const auto& c : lhs[j].coef) {
            if (c.second != 0) want[c.first] = c.second;
          }
          ok = ok && renamed == want;
        }
      });
    }
    return ok;
  }

  // --- whole stage ----------------------------------------------------------------------------
  void plan(int64_t& ldsBudgetBytes) {
    for (const auto& s : st_.stmts) {
      if (!s.redVars.empty()) {
        planPromotions(s, ldsBudgetBytes);
        break;
      }
    }
  }

  // Declares i_<v> (and p_<v>) for every variable of `group` from the flattened position `pos`
  // inside the block tile (row-major over the group's tile extents, last variable fastest) and
  // returns the predicate "position exists".
  std::string decodeGroup(const std::vector<std::string>& group, const std::string& pos, bool clamp = false) {
    int64_t total = 1;
    for (const auto& n : group) total *= var(n).tile;
    std::string pred = pos + " < " + std::to_string(total);
    // clamped: positions past the end alias the last valid one, so that addresses computed from
    // the decoded indices are always legal (used for operands whose surplus lanes are discarded)
    std::string src = pos;
    if (clamp) {
      src = "pc" + std::to_string(clampId_++) + "_";
      em_.line("const int " + src + " = min(" + pos + ", " + std::to_string(total - 1) + ");");
    }
    int64_t div = total;
    for (const auto& n : group) {
      const LoopVar& v = var(n);
      div /= v.tile;
      std::string e = src;
      if (div > 1) e = "(" + e + " / " + std::to_string(div) + ")";
      if (&n != &group.front()) e = e + " % " + std::to_string(v.tile);
      std::string base = std::to_string(v.min);
      if (v.numTiles > 1) base += " + " + tv(v) + " * " + std::to_string(v.tile);
      em_.line("const int p_" + v.name + " = " + e + ";");
      if (clamp && v.partial()) {
        em_.line("const int " + iv(v) + " = min(" + base + " + p_" + v.name + ", " + std::to_string(v.min + v.extent - 1) + ");");
      } else {
        em_.line("const int " + iv(v) + " = " + base + " + p_" + v.name + ";");
      }
      if (v.partial()) pred += " && " + base + " + p_" + v.name + " <= " + std::to_string(v.min + v.extent - 1);
    }
    return pred;
  }

  void emitMfma() {
    const StageStmt& s = st_.stmts[0];
    auto tileProduct = [&](const std::vector<std::string>& g) {
      int64_t t = 1;
      for (const auto& n : g) t *= var(n).tile;
      return t;
    };
    int64_t MT = tileProduct(st_.mfmaM), NT = tileProduct(st_.mfmaN), BT = tileProduct(st_.mfmaBatch),
            KT = tileProduct(st_.mfmaK);
    int64_t numMT = ceilDiv(MT, 16), numNT = ceilDiv(NT, 16), ksteps = ceilDiv(KT, 4);
    (void)KT;
    int64_t tiles = BT * numMT * numNT;
    // predicates that are statically true need no code
    auto groupExact = [&](const std::vector<std::string>& g, int64_t total, int64_t granule) {
      bool exact = total % granule == 0;
      for (const auto& n : g) exact &= !var(n).partial();
      return exact;
    };
    const ExprRef& loadA = s.rhs->args[st_.mfmaSwapOperands ? 1 : 0]; // holds the M-side variables
    const ExprRef& loadB = s.rhs->args[st_.mfmaSwapOperands ? 0 : 1]; // holds the N-side variables
    em_.line("// matrix cores: " + std::to_string(tiles) + " tiles of 16x16 per block, " + std::to_string(ksteps) +
             " steps of v_mfma_f32_16x16x4_f32 each, " + std::to_string(st_.waves) + " wavefront(s)");
    // (the register-resident operand is requested first: its latency overlaps the LDS staging)
    em_.line("const int lm_ = threadIdx.x & 15, lj_ = threadIdx.x >> 4;");
    // Lane group lj_ (0..3) owns a contiguous quarter of the flattened reduction and step ks_
    // walks inside it: when a quarter is a whole number of inner-variable periods, the inner
    // reduction indices of a step are compile-time constants after unrolling and only the
    // outermost one depends on the lane, so operand addresses become "lane base + immediate".
    const int64_t quarter = ceilDiv(KT, 4);
    ksteps = quarter;
    int64_t innerProd = 1;
    for (size_t i = 1; i < st_.mfmaK.size(); ++i) innerProd *= var(st_.mfmaK[i]).tile;
    const bool aligned = quarter % innerProd == 0;
    // Opens the loop over the reduction steps of a lane, decodes the reduction indices of the
    // step and declares kok_ when surplus steps exist; returns whether it did.
    auto openSteps = [&]() {
      em_.line(ksteps <= 128 ? "#pragma unroll" : "#pragma unroll 4");
      em_.open("for (int ks_ = 0; ks_ < " + std::to_string(ksteps) + "; ++ks_)");
      std::string kok;
      if (aligned) {
        int64_t div = innerProd;
        for (size_t i = 0; i < st_.mfmaK.size(); ++i) {
          const LoopVar& v = var(st_.mfmaK[i]);
          std::string e;
          if (i == 0) {
            e = "lj_ * " + std::to_string(quarter / innerProd) + " + ks_ / " + std::to_string(innerProd);
          } else {
            div /= v.tile;
            e = "(ks_ / " + std::to_string(div) + ") % " + std::to_string(v.tile);
          }
          // the surplus steps of the last lane group would decode past the outermost extent
          if (i == 0 && quarter * 4 != KT) e = "min(" + e + ", " + std::to_string(v.tile - 1) + ")";
          em_.line("const int p_" + v.name + " = " + e + ";");
          std::string base = std::to_string(v.min);
          if (v.numTiles > 1) base += " + " + tv(v) + " * " + std::to_string(v.tile);
          em_.line("const int " + iv(v) + " = " + base + " + p_" + v.name + ";");
        }
        if (quarter * 4 != KT) kok = "lj_ * " + std::to_string(quarter) + " + ks_ < " + std::to_string(KT);
      } else {
        em_.line("const int kk_ = lj_ * " + std::to_string(quarter) + " + ks_;");
        kok = decodeGroup(st_.mfmaK, "kk_", true);
        if (quarter * 4 == KT) kok.clear();
      }
      if (!kok.empty()) em_.line("const bool kok_ = " + kok + ";");
      return !kok.empty();
    };
    // surplus reduction steps must contribute exact zeros
    auto operandValue = [&](const ExprRef& load, bool masked) {
      std::string text = loadStr(load, "");
      return masked ? "(kok_ ? " + text + " : 0.0f)" : text;
    };
    const bool resident = mfmaKeepsMOperandInRegisters();
    if (resident) {
      em_.line("float am_[" + std::to_string(ksteps) + "];");
      em_.open("");
      em_.line("const int mt_ = 0, bt_ = 0;");
      em_.line("(void)mt_; (void)bt_;");
      if (!st_.mfmaBatch.empty()) decodeGroup(st_.mfmaBatch, "bt_", true);
      em_.line("const int mposa_ = lm_;");
      decodeGroup(st_.mfmaM, "mposa_", true);
      // consecutive steps of a lane read consecutive elements when the operand's reduction
      // subscripts are jointly contiguous: four steps are then fetched with one 16-byte load
      bool contiguous = aligned && quarter * 4 == KT && ksteps % 4 == 0;
      {
        Affine fa = flatAffine(loadA->name, loadA->args);
        contiguous &= fa.valid;
        int64_t expect = 1;
        for (size_t i = st_.mfmaK.size(); contiguous && i-- > 0;) {
          const LoopVar& v = var(st_.mfmaK[i]);
          contiguous &= fa.coefOf(v.name) == expect;
          expect *= v.tile;
        }
      }
      if (contiguous) {
        em_.line("#pragma unroll");
        em_.open("for (int kv_ = 0; kv_ < " + std::to_string(ksteps / 4) + "; ++kv_)");
        em_.line("const int ks_ = 4 * kv_;");
        int64_t div = innerProd;
        for (size_t i = 0; i < st_.mfmaK.size(); ++i) {
          const LoopVar& v = var(st_.mfmaK[i]);
          std::string e;
          if (i == 0) {
            e = "lj_ * " + std::to_string(quarter / innerProd) + " + ks_ / " + std::to_string(innerProd);
          } else {
            div /= v.tile;
            e = "(ks_ / " + std::to_string(div) + ") % " + std::to_string(v.tile);
          }
          em_.line("const int " + iv(v) + " = " + std::to_string(v.min) + " + " + e + ";");
        }
        em_.line("const __tc::floatx4 v_ = *(const __tc::floatx4u*)&p" + loadA->name + "[" +
                 flatIndex(loadA->name, loadA->args, "") + "];");
        em_.line("am_[ks_] = v_[0]; am_[ks_ + 1] = v_[1]; am_[ks_ + 2] = v_[2]; am_[ks_ + 3] = v_[3];");
        em_.close();
      } else {
        bool masked = openSteps();
        em_.line("am_[ks_] = " + operandValue(loadA, masked) + ";");
        em_.close();
      }
      em_.close();
    }
    // Epilogue operands that do not depend on the column (a bias per output row, say) are the
    // same for every tile of the wavefront: fetched once, ahead of the tile loop.
    hoistedLoads_.clear();
    if (resident) {
      std::vector<std::pair<std::string, ExprRef>> invariant;
      for (size_t i = 1; i < st_.stmts.size(); ++i) {
        visitUnconditional(st_.stmts[i].rhs, [&](const ExprRef& e) {
          if (e->kind != Expr::Load || e->name == st_.tensor || st_.views.at(e->name).isOutput) return;
          Affine fa = flatAffine(e->name, e->args);
          bool ok = fa.valid;
          for (const auto& n : st_.mfmaN) ok = ok && fa.coefOf(n) == 0;
          if (!ok) return;
          std::string text = "p" + e->name + "[" + flatIndex(e->name, e->args, "") + "]";
          for (const auto& h : invariant) {
            if (h.first == text) return;
          }
          invariant.emplace_back(text, e);
        });
      }
      if (!invariant.empty()) {
        for (size_t h = 0; h < invariant.size(); ++h) {
          em_.line(st_.views.at(invariant[h].second->name).type.cName() + " eh" + std::to_string(h) + "_[4];");
        }
        em_.line("#pragma unroll");
        em_.open("for (int r_ = 0; r_ < 4; ++r_)");
        em_.line("const int bt_ = 0, mpos_ = 4 * lj_ + r_;");
        em_.line("(void)bt_;");
        if (!st_.mfmaBatch.empty()) decodeGroup(st_.mfmaBatch, "bt_", true);
        decodeGroup(st_.mfmaM, "mpos_", true);
        for (size_t h = 0; h < invariant.size(); ++h) {
          em_.line("eh" + std::to_string(h) + "_[r_] = " + invariant[h].first + ";");
        }
        em_.close();
        for (size_t h = 0; h < invariant.size(); ++h) {
          hoistedLoads_[invariant[h].first] = "eh" + std::to_string(h) + "_[r_]";
        }
      }
    }
    // Reduction tiling: the outermost reduction variable may run over several tiles; operands
    // staged per reduction tile are copied inside that loop and the accumulators of all output
    // tiles of a wavefront live in registers across it.
    const LoopVar& k0 = var(st_.mfmaK[0]);
    const bool kTiled = k0.numTiles > 1;
    const int64_t tilesPerWave = ceilDiv(tiles, st_.waves);
    auto stagePromotions = [&](bool inside) {
      bool any = false;
      for (const auto& p : st_.promotions) any |= p.insideReductionTiles == inside;
      if (!any) return;
      if (suppressCopy && !inside) {
        for (const auto& p : st_.promotions) {
          if (p.insideReductionTiles) continue;
          declareLows(p);
          activePromotions_.insert(p.tensor);
        }
        return;
      }
      em_.line("__syncthreads();");
      for (const auto& p : st_.promotions) {
        if (p.insideReductionTiles != inside) continue;
        emitCopyIn(p);
        activePromotions_.insert(p.tensor);
      }
      em_.line("__syncthreads();");
    };
    // decodes the output tile tl_ of this wavefront: batch and column indices, nok_
    auto decodeTile = [&]() {
      em_.line("const int nt_ = tl_ % " + std::to_string(numNT) + ", mt_ = (tl_ / " + std::to_string(numNT) + ") % " +
               std::to_string(numMT) + ", bt_ = tl_ / " + std::to_string(numNT * numMT) + ";");
      // A row of the product depends on one row of the M-side operand only and a column on one
      // column of the N-side operand, so lanes past the end of a partial tile may load any legal
      // element (clamped indices): their results are never stored.
      std::string bok = st_.mfmaBatch.empty() ? "true" : decodeGroup(st_.mfmaBatch, "bt_", true);
      em_.line("const bool bok_ = " + bok + ";");
      em_.line("const int npos_ = nt_ * 16 + lm_;");
      em_.line("const bool nok_ = bok_ && " + decodeGroup(st_.mfmaN, "npos_", true) + ";");
      em_.line("(void)nok_;");
    };
    // existing output values when the statement accumulates into them
    auto loadExisting = [&](const std::string& acc) {
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int mpos_ = mt_ * 16 + 4 * lj_ + r_;");
      em_.line("const bool mok_ = " + decodeGroup(st_.mfmaM, "mpos_") + ";");
      em_.line("if (nok_ && mok_) " + acc + "[r_] = p" + st_.tensor + "[" + flatIndex(st_.tensor, st_.lhsSubs, "") + "];");
      em_.close();
    };
    // the reduction steps of the current reduction tile into accumulator `acc`
    auto multiply = [&](const std::string& acc) {
      em_.open("");
      em_.line("const int mposa_ = mt_ * 16 + lm_;");
      em_.line("const bool moka_ = bok_ && " + decodeGroup(st_.mfmaM, "mposa_", true) + ";");
      em_.line("(void)moka_;");
      bool masked = openSteps();
      em_.line("const float a_ = " + (resident ? std::string("am_[ks_]") : operandValue(loadA, masked)) + ";");
      em_.line("const float b_ = " + operandValue(loadB, masked) + ";");
      em_.line(acc + " = __builtin_amdgcn_mfma_f32_16x16x4f32(a_, b_, " + acc + ", 0, 0, 0);");
      em_.close();
      em_.close();
    };
    // Epilogue and store: a lane holds rows 4*lj_ .. 4*lj_+3 of column lm_.  Indices are clamped
    // to legal points, so the epilogue's loads need no guard: the four rows are finished first
    // (their loads issue together and, when they do not depend on the column, move out of the
    // tile loop), then stored under one test of the column.
    auto finish = [&](const std::string& acc) {
      const bool mExact = groupExact(st_.mfmaM, MT, 16);
      em_.line(accType_.cName() + " out_[4];");
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int mpos_ = mt_ * 16 + 4 * lj_ + r_;");
      decodeGroup(st_.mfmaM, "mpos_", true);
      em_.line(accType_.cName() + " acc_[1];");
      em_.line("acc_[0] = " + acc + "[r_];");
      outerPred_ = "";
      accValid_ = true;
      for (size_t i = 1; i < st_.stmts.size(); ++i) {
        const StageStmt& e = st_.stmts[i];
        if (e.op != ReduceOp::None) {
          int n = openUnrolled();
          em_.line("acc_[a_] = " + combine(e.op, "acc_[a_]", castTo(e.rhs, accType_, "acc_[a_]")) + ";");
          closeN(n);
        } else {
          emitPointwise(e);
        }
      }
      em_.line("out_[r_] = acc_[0];");
      em_.close();
      em_.open("if (nok_)");
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int mpos_ = mt_ * 16 + 4 * lj_ + r_;");
      std::string mok = decodeGroup(st_.mfmaM, "mpos_", true);
      em_.line(storeStmt(mExact ? "true" : mok, "out_[r_]"));
      em_.close();
      em_.close();
    };
    // which wavefront takes the surplus tile rotates with the block, so that the blocks sharing a
    // compute unit load its four SIMDs evenly
    const std::string waveRotation =
        "const int wv_ = (threadIdx.y + blockIdx.x + blockIdx.y + blockIdx.z) % " + std::to_string(st_.waves) + ";";
    int opened = 0;
    em_.open("");
    ++opened;
    stagePromotions(false);
    if (!kTiled) {
      em_.line(waveRotation);
      em_.open("for (int tl_ = wv_; tl_ < " + std::to_string(tiles) + "; tl_ += " + std::to_string(st_.waves) + ")");
      ++opened;
      decodeTile();
      em_.line("__tc::floatx4 c_ = {0.0f, 0.0f, 0.0f, 0.0f};");
      if (!s.init) loadExisting("c_");
      multiply("c_");
      finish("c_");
    } else {
      em_.line(waveRotation);
      em_.line("__tc::floatx4 cacc_[" + std::to_string(tilesPerWave) + "];");
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
      em_.line("cacc_[j_] = __tc::floatx4{0.0f, 0.0f, 0.0f, 0.0f};");
      if (!s.init) {
        em_.line("const int tl_ = wv_ + j_ * " + std::to_string(st_.waves) + ";");
        em_.open("if (tl_ < " + std::to_string(tiles) + ")");
        decodeTile();
        loadExisting("cacc_[j_]");
        em_.close();
      }
      em_.close();
      // Software pipeline over the reduction tiles (prefetchShared): the global loads of the next
      // tile's operands are issued before the current tile is multiplied and land in registers;
      // they go to LDS after the multiplication, between two barriers.
      bool pipelineK = kc_.opts.prefetchSharedValue;
      int64_t stagingRegs = 0;
      bool anyInside = false;
      for (const auto& p : st_.promotions) {
        if (!p.insideReductionTiles) continue;
        anyInside = true;
        stagingRegs += copyRegisters(p);
      }
      pipelineK = pipelineK && anyInside && stagingRegs <= 64;
      const std::string tk = tv(k0);
      if (pipelineK) {
        em_.open("");
        ++opened;
        for (const auto& p : st_.promotions) {
          if (p.insideReductionTiles) em_.line(copyRegisterDecl(p, "pk_" + p.tensor + "_"));
        }
        em_.open("");
        em_.line("const int " + tk + " = 0;");
        for (const auto& p : st_.promotions) {
          if (!p.insideReductionTiles) continue;
          declareLows(p);
          emitCopyLoads(p, "pk_" + p.tensor + "_");
        }
        em_.line("__syncthreads();");
        for (const auto& p : st_.promotions) {
          if (p.insideReductionTiles) emitCopyStores(p, "pk_" + p.tensor + "_");
        }
        em_.close();
      }
      em_.open("for (int " + tk + " = 0; " + tk + " < " + std::to_string(k0.numTiles) + "; ++" + tk + ")");
      if (pipelineK) {
        em_.line("__syncthreads();");
        em_.line("const bool more_ = " + tk + " + 1 < " + std::to_string(k0.numTiles) + ";");
        em_.open("if (more_)");
        tileOverride[k0.name] = "(" + tk + " + 1)";
        for (const auto& p : st_.promotions) {
          if (!p.insideReductionTiles) continue;
          declareLows(p);
          emitCopyLoads(p, "pk_" + p.tensor + "_");
        }
        tileOverride.clear();
        em_.close();
        for (const auto& p : st_.promotions) {
          if (!p.insideReductionTiles) continue;
          declareLows(p);
          activePromotions_.insert(p.tensor);
        }
      } else {
        stagePromotions(true);
      }
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
      em_.line("const int tl_ = wv_ + j_ * " + std::to_string(st_.waves) + ";");
      em_.open("if (tl_ < " + std::to_string(tiles) + ")");
      decodeTile();
      multiply("cacc_[j_]");
      em_.close();
      em_.close();
      if (pipelineK) {
        em_.line("__syncthreads();");
        em_.open("if (more_)");
        for (const auto& p : st_.promotions) {
          if (p.insideReductionTiles) emitCopyStores(p, "pk_" + p.tensor + "_");
        }
        em_.close();
      }
      em_.close();
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
      ++opened;
      em_.line("const int tl_ = wv_ + j_ * " + std::to_string(st_.waves) + ";");
      em_.open("if (tl_ < " + std::to_string(tiles) + ")");
      ++opened;
      decodeTile();
      finish("cacc_[j_]");
    }
    closeN(opened);
    hoistedLoads_.clear();
    for (const auto& p : st_.promotions) activePromotions_.erase(p.tensor);
  }

  void emit() {
    accType_ = st_.views.at(st_.tensor).type;
    em_.line("// stage " + std::to_string(stageIdx_) + ": " + st_.tensor);
    if (st_.mfma) {
      em_.open("");
      int openedTiles = 1;
      for (int i = kc_.k.sharedDepth; i < st_.numParallel; ++i) {
        const LoopVar& v = st_.vars[i];
        if (v.numTiles > 1) {
          em_.open("for (int t_" + v.name + " = 0; t_" + v.name + " < " + std::to_string(v.numTiles) + "; ++t_" + v.name + ")");
          ++openedTiles;
        }
      }
      emitMfma();
      closeN(openedTiles);
      return;
    }
    em_.open("");
    int opened = 1;
    // sequential tile loops of parallel variables not handled at kernel level
    for (int i = kc_.k.sharedDepth; i < st_.numParallel; ++i) {
      const LoopVar& v = st_.vars[i];
      if (v.numTiles > 1) {
        em_.open("for (int t_" + v.name + " = 0; t_" + v.name + " < " + std::to_string(v.numTiles) + "; ++t_" + v.name + ")");
        ++opened;
      }
    }
    // per-thread point loops that stay loops
    outerPred_ = idleAxesPredForCompute();
    for (int i = 0; i < st_.numParallel; ++i) {
      const LoopVar& v = st_.vars[i];
      if (v.unrolled) continue;
      std::string t = openPointLoop(v, false);
      ++opened;
      if (!t.empty()) outerPred_ += (outerPred_.empty() ? "" : " && ") + t;
    }
    em_.line(accType_.cName() + " acc_[" + std::to_string(st_.accCount) + "];");
    if (st_.threadReduction) em_.line(accType_.cName() + " part_[" + std::to_string(st_.accCount) + "];");
    accValid_ = false;
    int64_t budget = kc_.opts.generic.hasUnroll ? static_cast<int64_t>(kc_.opts.generic.unrollValue) : 1;
    for (const auto& s : st_.stmts) {
      if (s.redVars.empty()) {
        if (s.op != ReduceOp::None) {
          // reduction operator without reduction indices: a single combine with the old value
          if (!accValid_) preloadAcc();
          int n = openUnrolled();
          em_.line("acc_[a_] = " + combine(s.op, "acc_[a_]", castTo(s.rhs, accType_, "acc_[a_]")) + ";");
          closeN(n);
        } else {
          if (!accValid_ && readsOwnValue(s, st_)) preloadAcc();
          emitPointwise(s);
          accValid_ = true;
        }
      } else {
        emitReduction(s, budget);
      }
    }
    // store
    {
      int n = openUnrolled();
      std::string cond = "ok_";
      if (st_.threadReduction) cond += " && threadIdx.x == 0";
      em_.line(storeStmt(cond, "acc_[a_]"));
      closeN(n);
    }
    closeN(opened);
  }

  std::string idleAxesPredForCompute() const {
    // With a thread-mapped reduction all threads must take part in the barriers; idle axes are
    // filtered by the predicate rather than by skipping code.
    return idleAxesPred();
  }

 private:
  KernelCtx& kc_;
  StagePlan& st_;
  int stageIdx_;
  Emitter& em_;
  ScalarType accType_;
  bool accValid_ = false;
  std::string outerPred_;
  std::set<std::string> activePromotions_;
  std::map<std::string, std::string> hoistedLoads_; // printed global load -> register holding it
  bool inCachedReduction_ = false;
  std::string cacheSlot_;
  int clampId_ = 0;
};

// ------------------------------------------------------------------------------------------
// mapping of one kernel
// ------------------------------------------------------------------------------------------
void mapKernel(KernelCtx& kc, const DeviceLimits& limits) {
  const HipMappingOptions& o = kc.opts;
  KernelPlan& k = kc.k;
  TC_CHECK(!o.generic.hasTiling || !o.generic.tiling.empty()) << "tiling must hold at least one size";
  for (size_t a = 0; a < 3; ++a) {
    TC_CHECK_GT(o.grid[a], 0u) << "NYI: mapping to 0 blocks";
    TC_CHECK_GT(o.block[a], 0u) << "NYI: mapping to 0 threads";
  }
  std::array<int64_t, 3> blockUse{{1, 1, 1}}, gridUse{{1, 1, 1}};
  // Threads the stages may spread over.  A matrix-core stage addresses its lanes as
  // (threadIdx.x = lane of a wavefront, threadIdx.y = wavefront), so a kernel that holds one runs
  // 64 x waves threads and its other stages map onto that shape.
  std::array<int64_t, 3> blk{{static_cast<int64_t>(o.block[0]), static_cast<int64_t>(o.block[1]),
                              static_cast<int64_t>(o.block[2])}};
  int nb = static_cast<int>(o.block.size());
  int64_t waves = std::max<int64_t>(1, std::min<int64_t>(16, blk[0] * blk[1] * blk[2] / 64));
  for (const auto& st : k.stages) {
    if (st.mfma) {
      blk = {{64, waves, 1}};
      nb = 2;
    }
  }
  for (auto& st : k.stages) {
    // tile sizes by band position (lanes do not take a position)
    int pos = 0;
    for (auto& v : st.vars) {
      if (v.vectorLane) {
        v.tile = v.extent;
        v.numTiles = 1;
        continue;
      }
      int64_t t = 0;
      if (o.generic.hasTiling && pos < static_cast<int>(o.generic.tiling.size())) {
        t = static_cast<int64_t>(o.generic.tiling[pos]);
      }
      ++pos;
      // a lane-split variable is tiled in units of whole lane groups
      const LoopVar* next = (&v + 1 < &st.vars[0] + st.vars.size()) ? &v + 1 : nullptr;
      if (next && next->vectorLane && t > 0) t = std::max<int64_t>(1, t / next->extent);
      v.tile = (t <= 0 || t > v.extent) ? v.extent : t;
      v.numTiles = ceilDiv(v.extent, v.tile);
    }
    // blocks: outermost shared parallel variables, x first
    int axis = 0;
    for (int i = 0; i < st.numParallel && i < k.sharedDepth && axis < static_cast<int>(o.grid.size()); ++i) {
      LoopVar& v = st.vars[i];
      // a variable with a single tile has nothing to distribute and does not use up an axis
      if (v.vectorLane || v.numTiles == 1) continue;
      v.blockAxis = axis;
      v.gridExtent = std::min<int64_t>(static_cast<int64_t>(o.grid[axis]), v.numTiles);
      gridUse[axis] = std::max(gridUse[axis], v.gridExtent);
      ++axis;
    }
    if (st.mfma) {
      // one wavefront per 16x16 output tile; the block holds as many wavefronts as the block
      // option has threads.  Only the outermost reduction variable may be tiled (its tile must
      // divide the extent): operands are then staged in LDS one reduction tile at a time while the
      // accumulators of a wavefront's output tiles stay in registers.
      bool firstReduction = true;
      for (auto& v : st.vars) {
        if (!v.reduction) continue;
        bool keep = firstReduction && v.numTiles > 1 && v.extent % v.tile == 0;
        firstReduction = false;
        if (!keep) {
          v.tile = v.extent;
          v.numTiles = 1;
        }
      }
      st.waves = waves;
      blockUse[0] = std::max<int64_t>(blockUse[0], 64);
      blockUse[1] = std::max<int64_t>(blockUse[1], st.waves);
      continue;
    }
    // threads: innermost variables, x first
    bool hasReduction = false;
    for (const auto& s : st.stmts) hasReduction |= !s.redVars.empty();
    st.threadReduction = o.generic.matchLibraryCallsValue && hasReduction && blk[0] > 1 && o.block[0] > 1;
    int taxis = 0;
    if (st.threadReduction) {
      for (int i = static_cast<int>(st.vars.size()) - 1; i >= st.numParallel; --i) {
        if (!st.vars[i].vectorLane) {
          st.vars[i].threadAxis = 0;
          break;
        }
      }
      taxis = 1;
    }
    for (int i = st.numParallel - 1; i >= 0 && taxis < nb; --i) {
      if (st.vars[i].vectorLane) continue;
      st.vars[i].threadAxis = taxis++;
    }
    for (auto& v : st.vars) {
      if (v.threadAxis >= 0) {
        int64_t want = v.tile;
        if (st.threadReduction && v.reduction) {
          // the reduction library is fastest on rows that are lane groups of a wavefront or
          // whole wavefronts: tighten to the next such width when the option allows it
          if (want <= 64) {
            while (want & (want - 1)) ++want;
          } else {
            want = ceilDiv(want, 64) * 64;
          }
          if (want > blk[v.threadAxis]) want = v.tile;
        }
        blockUse[v.threadAxis] = std::max(blockUse[v.threadAxis], std::min<int64_t>(blk[v.threadAxis], want));
      }
    }
  }
  // XCD-aware block order.  Consecutive linear block ids go round-robin to the 8 XCDs, each
  // with its own L2: blocks that differ only in the x-mapped tile index end up on different XCDs.
  // Operands that do not depend on a block-mapped variable are shared by the blocks along it, so
  // the variable with the least shared bytes takes blockIdx.x and the one with the most the
  // slowest axis (its blocks then meet in one L2 when the faster extents are multiples of 8).
  {
    const StagePlan& s0 = k.stages.front();
    std::vector<int> positions;
    for (int i = 0; i < s0.numParallel && i < k.sharedDepth; ++i) {
      if (s0.vars[i].blockAxis >= 0) positions.push_back(i);
    }
    if (positions.size() >= 2) {
      std::vector<double> shared(positions.size(), 0.0);
      for (const auto& st : k.stages) {
        std::map<std::string, std::set<std::string>> uses; // tensor -> variables in its subscripts
        for (const auto& stmt : st.stmts) {
          visit(stmt.rhs, [&](const ExprRef& e) {
            if (e->kind != Expr::Load) return;
            auto& u = uses[e->name];
            for (const auto& a : e->args) {
              Affine x = ir::toAffine(a);
              if (!x.valid) {
                for (const auto& v : st.vars) u.insert(v.name); // unknown: assume it depends on all
                continue;
              }
              for (const auto& c : x.coef) {
                if (c.second != 0) u.insert(c.first);
              }
            }
          });
        }
        for (const auto& t : uses) {
          const TensorView& view = st.views.at(t.first);
          double bytes = view.type.bytes();
          for (auto e : view.extents) bytes *= static_cast<double>(e);
          for (int pos : positions) {
            if (t.second.count(st.vars[pos].name)) bytes /= static_cast<double>(st.vars[pos].numTiles);
          }
          for (size_t r = 0; r < positions.size(); ++r) {
            if (!t.second.count(st.vars[positions[r]].name)) shared[r] += bytes;
          }
        }
      }
      std::vector<size_t> order(positions.size());
      for (size_t r = 0; r < order.size(); ++r) order[r] = r;
      std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return shared[a] < shared[b]; });
      bool changes = false;
      for (size_t r = 0; r < order.size(); ++r) changes |= order[r] != r;
      // every stage must distribute the same positions over the same extents
      bool uniform = true;
      for (const auto& st : k.stages) {
        int mapped = 0;
        for (int i = 0; i < st.numParallel; ++i) mapped += st.vars[i].blockAxis >= 0;
        uniform &= mapped == static_cast<int>(positions.size());
        for (int pos : positions) {
          uniform &= pos < st.numParallel && st.vars[pos].blockAxis == s0.vars[pos].blockAxis &&
              st.vars[pos].gridExtent == s0.vars[pos].gridExtent;
        }
      }
      if (changes && uniform && s0.vars[positions[order[0]]].gridExtent % 8 == 0) {
        gridUse = {{1, 1, 1}};
        for (auto& st : k.stages) {
          for (size_t r = 0; r < order.size(); ++r) {
            LoopVar& v = st.vars[positions[order[r]]];
            v.blockAxis = static_cast<int>(r);
            gridUse[r] = std::max(gridUse[r], v.gridExtent);
          }
        }
      }
    }
  }
  k.block = blockUse;
  k.grid = gridUse;
  TC_CHECK_LE(k.block[0] * k.block[1] * k.block[2], limits.maxThreadsPerBlock)
      << "thread block of " << k.block[0] << "x" << k.block[1] << "x" << k.block[2] << " exceeds the device limit";
  int64_t budget = o.generic.hasUnroll ? static_cast<int64_t>(o.generic.unrollValue) : 1;
  for (auto& st : k.stages) {
    for (auto& v : st.vars) {
      v.perThread = v.threadAxis >= 0 ? ceilDiv(v.tile, k.block[v.threadAxis]) : v.tile;
    }
    if (st.mfma) {
      st.accCount = 1;
      continue;
    }
    // register tile: innermost parallel variables first, while the tile fits the budget
    int64_t prod = 1;
    for (int i = st.numParallel - 1; i >= 0; --i) {
      LoopVar& v = st.vars[i];
      if (v.vectorLane || prod * v.perThread <= std::max<int64_t>(budget, 1) || v.perThread == 1) {
        // bound on fully unrolled code: every accumulator of a thread-mapped reduction also
        // unrolls one block reduction (compile time of hipRTC grows steeply beyond this)
        if (prod * v.perThread > (st.threadReduction ? 32 : 256)) break;
        v.unrolled = true;
        prod *= v.perThread;
      } else {
        break;
      }
    }
    st.accCount = prod;
  }
}

std::string kernelSignature(const ir::Function& f, const std::string& name, int64_t nt) {
  std::ostringstream ss;
  ss << "extern \"C\" __global__ void __launch_bounds__(" << nt << ") " << name << "(";
  bool first = true;
  for (const auto& p : f.params) {
    ss << (first ? "" : ", ") << "int " << p.first;
    first = false;
  }
  for (const auto& t : f.outputs) {
    ss << (first ? "" : ", ") << t.type.cName() << "* __restrict__ p" << t.name;
    first = false;
  }
  for (const auto& t : f.inputs) {
    ss << (first ? "" : ", ") << "const " << t.type.cName() << "* __restrict__ p" << t.name;
    first = false;
  }
  ss << ")";
  return ss.str();
}

void emitKernel(KernelCtx& kc, const DeviceLimits& limits, Emitter& em) {
  KernelPlan& k = kc.k;
  std::vector<StageCodegen> gens;
  gens.reserve(k.stages.size());
  int64_t ldsBudget = limits.ldsBytesPerBlock;
  if (kc.opts.hasMaxSharedMemory) ldsBudget = std::min<int64_t>(ldsBudget, kc.opts.maxSharedMemoryValue);
  int64_t scratchElems = 0;
  ScalarType scratchType;
  for (auto& st : k.stages) {
    if (st.threadReduction) {
      int64_t bx = k.block[0], rows = k.block[1] * k.block[2];
      int64_t e = ((bx & (bx - 1)) == 0 && bx <= 64) ? 1 : (bx % 64 == 0 ? (bx / 64) * rows : bx * rows);
      scratchElems = std::max(scratchElems, e);
      ScalarType t = st.views.at(st.tensor).type;
      if (t.bytes() > scratchType.bytes() || scratchElems == e) scratchType = t;
    }
  }
  ldsBudget -= scratchElems * 8;
  int64_t before = ldsBudget;
  for (size_t i = 0; i < k.stages.size(); ++i) {
    gens.emplace_back(kc, k.stages[i], static_cast<int>(i), em);
    gens.back().plan(ldsBudget);
  }
  k.ldsBytes = (before - ldsBudget) + scratchElems * 8;

  // Register promotion across stages (usePrivateMemory): an input that several stages read with
  // the same loop structure and addresses is loaded once, by the first of them, into a
  // per-thread register array that lives across the stages of one block iteration.
  std::vector<std::string> cacheDecls;
  if (kc.opts.usePrivateMemoryValue && gens.size() >= 2) {
    std::vector<std::string> sigs(gens.size());
    std::vector<std::vector<std::pair<std::string, std::string>>> loads(gens.size());
    for (size_t i = 0; i < gens.size(); ++i) sigs[i] = gens[i].cacheSignature(loads[i]);
    std::map<std::string, std::string> produced; // canonical load -> cache name
    for (size_t i = 0; i < gens.size(); ++i) {
      if (sigs[i].empty() || sigs[i] != sigs[0]) continue;
      if (gens[i].cacheSlots() > 256) continue;
      for (const auto& l : loads[i]) {
        bool sharedLater = false;
        for (size_t j = 0; j < gens.size(); ++j) {
          if (j == i || sigs[j] != sigs[i]) continue;
          for (const auto& m : loads[j]) sharedLater |= m.first == l.first;
        }
        if (!sharedLater) continue;
        auto it = produced.find(l.first);
        bool producer = it == produced.end();
        if (producer) {
          std::string name = "rcache" + std::to_string(produced.size()) + "_";
          it = produced.emplace(l.first, name).first;
          std::string tensor = l.second.substr(1, l.second.find('[') - 1);
          cacheDecls.push_back(k.stages[i].views.at(tensor).type.cName() + " " + name + "[" +
                               std::to_string(gens[i].cacheSlots()) + "];");
        }
        gens[i].regCaches[l.second] = StageCodegen::RegCache{it->second, producer};
        gens[i].cachedStmt_ = gens[i].firstReduction();
      }
    }
  }

  // The same for a pointwise stage after a reduction over the same elements (normalise after
  // moments, say): when an operand's address forms agree, the reduction's single read of each
  // element fills the cache and the pointwise stage finds it there.
  if (kc.opts.usePrivateMemoryValue && gens.size() >= 2) {
    for (size_t j = 1; j < gens.size(); ++j) {
      const StagePlan& cs = k.stages[j];
      bool pointwise = !cs.mfma && !cs.threadReduction && gens[j].firstReduction() == nullptr;
      if (!pointwise) continue;
      for (const auto& stmt : cs.stmts) {
        if (stmt.op != ReduceOp::None) continue;
        visitUnconditional(stmt.rhs, [&](const ExprRef& e) {
          if (e->kind != Expr::Load) return;
          StageCodegen::AddressForm want = gens[j].addressForm(e, nullptr);
          if (!want.valid || want.slots > 256) return;
          std::string mine = "p" + e->name + "[" + gens[j].flatIndex(e->name, e->args, "") + "]";
          if (gens[j].regCaches.count(mine)) return;
          for (size_t i = 0; i < j; ++i) {
            const StageStmt* red = gens[i].firstReduction();
            if (!red || k.stages[i].mfma) continue;
            if (gens[i].cachedStmt_ && gens[i].cachedStmt_ != red) continue;
            std::string found;
            visitUnconditional(red->rhs, [&](const ExprRef& m) {
              if (m->kind != Expr::Load || !found.empty()) return;
              if (gens[i].addressForm(m, red) == want) {
                found = "p" + m->name + "[" + gens[i].flatIndex(m->name, m->args, "") + "]";
              }
            });
            if (found.empty()) continue;
            auto it = gens[i].regCaches.find(found);
            if (it == gens[i].regCaches.end()) {
              std::string name = "rcache" + std::to_string(cacheDecls.size()) + "_";
              cacheDecls.push_back(cs.views.at(e->name).type.cName() + " " + name + "[" + std::to_string(want.slots) + "];");
              it = gens[i].regCaches.emplace(found, StageCodegen::RegCache{name, true}).first;
              gens[i].cachedStmt_ = red;
            }
            gens[j].regCaches[mine] = StageCodegen::RegCache{it->second.name, false};
            gens[j].cachedPointwise_ = true;
            break;
          }
        });
      }
    }
  }

  em.open(kernelSignature(kc.f, k.name, kc.NT()));
  for (const auto& p : kc.f.params) em.line("(void)" + p.first + ";");
  em.line("const int tid_ = threadIdx.x + " + std::to_string(k.block[0]) + " * (threadIdx.y + " +
          std::to_string(k.block[1]) + " * threadIdx.z);");
  em.line("(void)tid_;");
  if (scratchElems > 0) {
    // one scratch area typed per use; sized for the widest element
    em.line("__shared__ double red_scratch_raw_[" + std::to_string(scratchElems) + "];");
  }
  for (auto& g : gens) g.emitLdsDecls();
  // kernel-level tile loops over the shared parallel variables (taken from the first stage):
  // first the tile indices that are plain block ids, then the loops, outermost first
  int opened = 0;
  const StagePlan& s0 = k.stages.front();
  std::vector<const LoopVar*> loops;
  for (int i = 0; i < k.sharedDepth && i < s0.numParallel; ++i) {
    const LoopVar& v = s0.vars[i];
    if (v.vectorLane || v.numTiles == 1) continue;
    if (v.blockAxis >= 0 && v.gridExtent == v.numTiles) {
      em.line("const int t_" + v.name + " = blockIdx." + axisName(v.blockAxis) + ";");
    } else {
      loops.push_back(&v);
    }
  }
  auto loopHeader = [&](const LoopVar& v, std::string& start, std::string& step) {
    start = v.blockAxis >= 0 ? std::string("blockIdx.") + axisName(v.blockAxis) : "0";
    step = v.blockAxis >= 0 ? std::to_string(v.gridExtent) : "1";
    std::string t = "t_" + v.name;
    return "for (int " + t + " = " + start + "; " + t + " < " + std::to_string(v.numTiles) + "; " + t + " += " + step + ")";
  };
  // Software pipeline over the innermost kernel-level loop (prefetchShared): the global loads of
  // the next tile's LDS footprints are issued before the current tile is computed and land in
  // registers; they are written to LDS after the computation, between two barriers.
  bool pipelined = false;
  if (kc.opts.prefetchSharedValue && k.stages.size() == 1 && !loops.empty() && !gens[0].promotions().empty()) {
    int64_t regs = 0;
    pipelined = true;
    for (const auto& p : gens[0].promotions()) {
      pipelined &= !p.insideReductionTiles;
      regs += gens[0].copyRegisters(p);
    }
    pipelined &= regs <= 96;
  }
  for (size_t li = 0; li < loops.size(); ++li) {
    const LoopVar& v = *loops[li];
    std::string start, step;
    std::string header = loopHeader(v, start, step);
    if (!(pipelined && li + 1 == loops.size())) {
      em.open(header);
      ++opened;
      continue;
    }
    StageCodegen& g = gens[0];
    std::string t = "t_" + v.name;
    em.open("");
    ++opened;
    for (const auto& p : g.promotions()) {
      em.line(g.copyRegisterDecl(p, "pf_" + p.tensor + "_"));
    }
    em.open("");
    em.line("const int " + t + " = " + start + ";");
    for (const auto& p : g.promotions()) {
      g.declareLows(p);
      g.emitCopyLoads(p, "pf_" + p.tensor + "_");
    }
    for (const auto& p : g.promotions()) g.emitCopyStores(p, "pf_" + p.tensor + "_");
    em.close();
    em.open(header);
    ++opened;
    em.line("__syncthreads();");
    em.line("const bool more_ = " + t + " + " + step + " < " + std::to_string(v.numTiles) + ";");
    em.open("if (more_)");
    g.tileOverride[v.name] = "(" + t + " + " + step + ")";
    for (const auto& p : g.promotions()) {
      g.declareLows(p);
      g.emitCopyLoads(p, "pf_" + p.tensor + "_");
    }
    g.tileOverride.clear();
    em.close();
    g.suppressCopy = true;
  }
  for (const auto& d : cacheDecls) em.line(d);
  // Barriers between the stages: only where a later stage touches what an earlier one wrote (or
  // overwrites what it read) through different threads, at the weakest sufficient level, placed
  // by the exact search of sync_placement.h.  Every stage writes elements indexed by the
  // kernel-level loop variables and reads other stages' results at the same indices, so nothing
  // is carried from one iteration of those loops to the next.
  std::vector<int> syncAfter(k.stages.size(), 0);
  {
    const int n = static_cast<int>(k.stages.size());
    SyncNeeds need(n, std::vector<int>(n, 0));
    const int level = static_cast<int>(kc.NT() <= limits.wavefront ? SyncLevel::Wave : SyncLevel::Block);
    for (int i = 0; i < n; ++i) {
      for (int j = i + 1; j < n; ++j) {
        const StagePlan& a = k.stages[i];
        const StagePlan& b = k.stages[j];
        bool conflict = a.tensor == b.tensor || tensorsRead(b).count(a.tensor) || tensorsRead(a).count(b.tensor);
        if (conflict && !gens[j].readsPrivatelyFrom(a)) need[i][j - i] = level;
      }
    }
    for (const auto& sy : findBestSyncs(need, opened > 0)) syncAfter[sy.first] = static_cast<int>(sy.second);
  }
  auto emitSync = [&](int level) {
    if (level == static_cast<int>(SyncLevel::Block)) {
      em.line("__syncthreads();");
    } else if (level == static_cast<int>(SyncLevel::Wave)) {
      // the block is a single wavefront: order its memory operations, no hardware barrier
      em.line("__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");");
      em.line("__builtin_amdgcn_wave_barrier();");
    }
  };
  for (size_t i = 0; i < k.stages.size(); ++i) {
    if (i > 0) emitSync(syncAfter[i - 1]);
    if (k.stages[i].threadReduction) {
      em.open("");
      em.line(k.stages[i].views.at(k.stages[i].tensor).type.cName() + "* red_scratch_ = (" +
              k.stages[i].views.at(k.stages[i].tensor).type.cName() + "*)red_scratch_raw_;");
      gens[i].emit();
      em.close();
    } else {
      gens[i].emit();
    }
  }
  if (pipelined) {
    StageCodegen& g = gens[0];
    em.line("__syncthreads();");
    em.open("if (more_)");
    for (const auto& p : g.promotions()) g.emitCopyStores(p, "pf_" + p.tensor + "_");
    em.close();
  }
  emitSync(syncAfter.back());
  for (int i = 0; i < opened; ++i) em.close();
  em.close();
}

} // namespace

MappedProgram mapToHip(
    const ir::Function& f,
    const HipMappingOptions& options,
    const std::string& specializedName,
    const DeviceLimits& limits) {
  for (const auto& t : f.outputs) {
    for (auto m : t.mins) {
      TC_CHECK_EQ(m, 0) << "output " << t.name << " has a non-zero inferred lower bound; not supported";
    }
  }
  // 1. stages
  std::vector<RawStage> raw;
  bool allowStageFusion = options.generic.intraTileScheduleOptions.fusionStrategy != FusionStrategy::Min ||
      options.generic.outerScheduleOptions.fusionStrategy != FusionStrategy::Min;
  for (const auto& s : f.statements) {
    for (const auto& subs : accessesTo(s, s.tensor)) {
      TC_CHECK(isIdentityAccess(subs, s.lhsVars))
          << "statement on " << s.tensor << " reads its own output at other points; not supported";
    }
    bool merged = false;
    if (!raw.empty() && allowStageFusion && sameBox(raw.back().first(), s)) {
      raw.back().stmts.push_back(&s);
      merged = true;
    }
    if (!merged) {
      RawStage r;
      r.stmts.push_back(&s);
      raw.push_back(r);
    }
  }
  // 2. kernels
  struct Group {
    std::vector<size_t> stages;
    int depth;
  };
  std::vector<Group> groups;
  FusionStrategy fs = options.generic.outerScheduleOptions.fusionStrategy;
  for (size_t i = 0; i < raw.size(); ++i) {
    bool joined = false;
    if (!groups.empty() && fs != FusionStrategy::Min) {
      Group& g = groups.back();
      int d = g.depth;
      for (size_t j : g.stages) {
        d = std::min(d, sharedPrefix(raw[j], raw[i]));
      }
      int need = 1;
      if (fs == FusionStrategy::Preserve3Coincident) {
        size_t rank = raw[i].first().lhsVars.size();
        for (size_t j : g.stages) rank = std::min(rank, raw[j].first().lhsVars.size());
        need = static_cast<int>(std::min<size_t>(3, rank));
      }
      if (d >= need && d >= 1) {
        g.stages.push_back(i);
        g.depth = d;
        joined = true;
      }
    }
    if (!joined) {
      groups.push_back(Group{{i}, static_cast<int>(raw[i].first().lhsVars.size())});
    }
  }
  // 3. plans
  MappedProgram prog;
  for (const auto& p : f.params) {
    prog.paramNames.push_back(p.first);
    prog.paramValues.push_back(p.second);
  }
  int64_t maxNumel = 0;
  for (const auto& t : f.inputs) maxNumel = std::max(maxNumel, t.numel());
  for (const auto& t : f.outputs) maxNumel = std::max(maxNumel, t.numel());
  TC_CHECK_LT(maxNumel, (1LL << 31)) << "tensors with 2^31 or more elements are not supported yet";

  bool anyThreadReduction = false;
  std::vector<std::unique_ptr<Emitter>> bodies;
  for (size_t gi = 0; gi < groups.size(); ++gi) {
    KernelPlan k;
    k.name = specializedName + (gi == 0 ? "" : "_k" + std::to_string(gi));
    bool single = groups[gi].stages.size() == 1;
    for (size_t si : groups[gi].stages) {
      StageBuilder b(f);
      b.init(raw[si]);
      if (options.collapseContiguousValue) b.collapse(single ? 0 : static_cast<size_t>(groups[gi].depth));
      k.stages.push_back(std::move(b.st));
    }
    k.sharedDepth = single ? k.stages[0].numParallel : groups[gi].depth;
    // later stages of a fused kernel adopt the first stage's names for the shared variables;
    // their other variables get a stage suffix so nothing can collide
    for (size_t si = 1; si < k.stages.size(); ++si) {
      StagePlan& st = k.stages[si];
      std::map<std::string, std::string> ren;
      for (size_t vi = 0; vi < st.vars.size(); ++vi) {
        ren[st.vars[vi].name] = static_cast<int>(vi) < k.sharedDepth
            ? k.stages[0].vars[vi].name
            : st.vars[vi].name + "_s" + std::to_string(si);
      }
      auto sub = [&](const ExprRef& e) -> ExprRef {
        return e->kind == Expr::Var ? mkVar(ren.at(e->name)) : nullptr;
      };
      for (auto& v : st.vars) v.name = ren.at(v.name);
      for (auto& e : st.lhsSubs) e = rewrite(e, sub);
      for (auto& ss : st.stmts) {
        ss.rhs = rewrite(ss.rhs, sub);
        for (auto& r : ss.redVars) r = ren.at(r);
      }
    }
    if (options.useMfmaValue) {
      for (auto& st : k.stages) classifyContraction(st);
    }
    // vector lanes on the variable that will sit on threadIdx.x
    if (options.vectorWidthValue > 1) {
      for (auto& st : k.stages) {
        if (st.mfma) continue;
        bool hasRed = false;
        for (const auto& s : st.stmts) hasRed |= !s.redVars.empty();
        bool threadRed = options.generic.matchLibraryCallsValue && hasRed && options.block[0] > 1;
        std::string target;
        if (threadRed) {
          target = st.vars.back().name;
        } else if (st.numParallel > 0) {
          target = st.vars[st.numParallel - 1].name;
        }
        // the shared prefix must keep its shape in every stage
        bool inPrefix = !threadRed && !single && st.numParallel - 1 < k.sharedDepth;
        if (!target.empty() && !inPrefix) {
          StageBuilder b(f);
          b.st = std::move(st);
          int before = b.st.numParallel;
          b.splitLanes(target, options.vectorWidthValue);
          if (single) k.sharedDepth += b.st.numParallel - before;
          st = std::move(b.st);
        }
      }
    }
    prog.kernels.push_back(std::move(k));
  }
  std::ostringstream src;
  for (auto& k : prog.kernels) {
    KernelCtx kc{f, options, k};
    mapKernel(kc, limits);
    for (const auto& st : k.stages) anyThreadReduction |= st.threadReduction;
    bodies.emplace_back(new Emitter());
    emitKernel(kc, limits, *bodies.back());
  }
  src << "// generated by the TC HIP mapper for gfx950; function " << f.name << "\n";
  src << hip::deviceLibrary(anyThreadReduction);
  for (const auto& b : bodies) src << "\n" << b->out.str();
  prog.source = src.str();
  return prog;
}

} // namespace mapper
} // namespace tc
