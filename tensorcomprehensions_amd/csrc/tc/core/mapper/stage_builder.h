// Part of mapper.cc: statements -> stages, stage canonicalisation (merging contiguous
// variables, vector lanes) and the classification of dense contractions.  Included once,
// inside the anonymous namespace of mapper.cc, after the expression helpers.
#pragma once

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

// Largest d such that the dependence between stages A (earlier) and B is point-wise in the
// first d left-hand-side positions of both, or -1 when they cannot share a kernel.
int sharedPrefix(const RawStage& A, const RawStage& B) {
  const ir::Statement &a0 = A.first(), &b0 = B.first();
  // partial sums of all blocks must be complete before anything reads them, and the zeroing must
  // be complete before the first of them arrives: a kernel of its own
  if (a0.atomic || b0.atomic) return -1;
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
  if (a0.tensor == b0.tensor && a0.lhsVars.size() > d) {
    // a later stage of another shape rewrites the tensor: they share a kernel only when every
    // subscript of the tensor is a shared variable (each iteration then touches its own element)
    return -1;
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
    st.atomic = s0.atomic;
    for (const auto& v : s0.lhsVars) {
      if (s0.sliceVar.empty() || v != s0.sliceVar) st.lhsSubs.push_back(mkVar(v));
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
      ss.init = s->init || s->atomic; // a partial sum starts from zero, the tensor is never read

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
    if (a.extent * b.extent >= (int64_t(1) << 31)) return false; // loop variables are 32-bit
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

// An operand of a product the matrix cores take: a load of a float tensor, or a load of a float16
// tensor converted to float (`float(A(m, r_k))`: every half is a float, and products of two
// halves are exact in float).  Null for anything else.
inline ExprRef contractionOperand(const ExprRef& e) {
  const ScalarType f32{ScalarType::Float, 32}, f16{ScalarType::Float, 16};
  if (e->kind == Expr::Load && e->type == f32) return e;
  if (e->kind == Expr::Cast && e->type == f32 && e->args.size() == 1 && e->args[0]->kind == Expr::Load && e->args[0]->type == f16) {
    return e->args[0];
  }
  return nullptr;
}

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
  if (e->kind != Expr::Binary || e->name != "*" || !contractionOperand(e->args[0]) || !contractionOperand(e->args[1])) {
    return false;
  }
  for (const auto& operand : e->args) {
    const ExprRef l = contractionOperand(operand);
    if (l->name == st.tensor) return false;
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

