// Part of mapper.cc: code generation for one stage of a kernel (LDS promotion and copies,
// point loops with folded points, reductions, matrix-core tiles, register caches).  Included
// once, inside the anonymous namespace of mapper.cc, after stage_builder.h.
#pragma once

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
  std::string idx = "int"; // type of non-affine subscript values inside an element offset
  // Some tensor has 2^31 or more elements: element offsets into global memory are formed in 64
  // bits (loop variables stay int: every extent is below 2^31).
  bool wide = false;
  bool kernelLoops = false; // the stages sit inside loops over tiles that the blocks share out
  // A tensor one stage of the kernel produces and later stages of the same kernel read: the part
  // a block produces during one kernel-level iteration is kept in LDS as well (the producer stores
  // every element to both places) and the readers take it from there instead of from memory.
  struct Forward {
    std::string ldsName;
    int producer = 0;
    std::vector<std::string> lows;   // origin of the block's box per view dimension, as C
    std::vector<int64_t> extents, strides;
    int64_t elems = 0;
  };
  std::map<std::string, Forward> forwards;
  // The result of a block-wide reduction that later stages of the kernel read at the element the
  // block has just produced: after the reduction every thread holds the value, so the readers take
  // it from a register instead of from memory (thread 0 still stores it for later kernels).  Later
  // stages that update the same element in place (mean(n) = mean(n) / K after the sum) work on the
  // register too, and only the last of the writers stores.
  struct RegisterForward {
    std::string name;
    int producer = 0;
    int lastWriter = 0;
  };
  std::map<std::string, RegisterForward> registerForwards;
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

  // affine over i_<var> values -> C; `wide`: every term is formed in 64 bits
  std::string affineStr(const Affine& a, bool wide = false) const {
    std::ostringstream ss;
    bool first = true;
    for (const auto& c : a.coef) {
      if (c.second == 0) continue;
      int64_t k = c.second;
      if (!first) ss << (k < 0 ? " - " : " + ");
      else if (k < 0) ss << "-";
      int64_t m = k < 0 ? -k : k;
      if (wide) {
        ss << "(int64)" << m << " * ";
      } else if (m != 1) {
        ss << m << " * ";
      }
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

  // Column sums.  While the body of an unrolled matrix-core tile loop is generated behind a cache
  // of column indices, the part of an element offset that depends on the N-side variables alone
  // (14 * i_h + 100352 * i_n + i_w of a store, 16 * i_h + i_w of an LDS read) is replaced by one
  // value per unrolled tile, ds<k>_[j_], which the pass ahead of the staging copy computes: the
  // multiplications leave the code behind the barrier.  Each distinct combination of coefficients
  // gets one such array.
  bool columnSums_ = false;
  std::vector<std::string> columnVars_;
  std::vector<Affine> columnCombos_;
  std::string columnSumOf(const Affine& part) {
    for (size_t k = 0; k < columnCombos_.size(); ++k) {
      bool same = true;
      for (const auto& n : columnVars_) same &= columnCombos_[k].coefOf(n) == part.coefOf(n);
      if (same) return "ds" + std::to_string(k) + "_[j_]";
    }
    columnCombos_.push_back(part);
    return "ds" + std::to_string(columnCombos_.size() - 1) + "_[j_]";
  }
  // moves the N-side terms of `a` (each scaled by `scale`) into `part`
  void takeColumnTerms(Affine& a, int64_t scale, Affine& part) const {
    for (const auto& n : columnVars_) {
      auto it = a.coef.find(n);
      if (it == a.coef.end() || it->second == 0) continue;
      part.coef[n] += it->second * scale;
      it->second = 0;
    }
  }
  static bool anyTerm(const Affine& a) {
    for (const auto& c : a.coef) {
      if (c.second != 0) return true;
    }
    return false;
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
    if (columnSums_ && !kc_.wide) {
      Affine part;
      part.valid = true;
      takeColumnTerms(total, 1, part);
      if (anyTerm(part)) return columnSumOf(part) + " + " + affineStr(total, false) + extra;
    }
    return affineStr(total, kc_.wide) + extra;
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

  // Box of elements of a tensor this stage touches through subscripts of one shape during one
  // kernel-level iteration: kernel-level variables span their tile, every other variable its
  // whole extent.  Origins are affine in the kernel-level tile indices (symbols "t_<var>").
  struct IterationBox {
    bool valid = false;
    std::vector<Affine> low;
    std::vector<int64_t> extents;
  };
  IterationBox iterationBox(const std::vector<std::vector<Affine>>& accesses) const {
    IterationBox box;
    if (accesses.empty()) return box;
    const auto& ref = accesses.front();
    for (const auto& a : accesses) {
      if (a.size() != ref.size()) return box;
      for (size_t j = 0; j < a.size(); ++j) {
        if (!a[j].valid || a[j].coef != ref[j].coef) return box;
      }
    }
    for (size_t j = 0; j < ref.size(); ++j) {
      int64_t lo = ref[j].constant, hi = ref[j].constant;
      for (const auto& a : accesses) {
        lo = std::min(lo, a[j].constant);
        hi = std::max(hi, a[j].constant);
      }
      Affine low;
      low.valid = true;
      low.constant = lo;
      int64_t ext = 1 + hi - lo;
      for (const auto& c : ref[j].coef) {
        if (c.second == 0) continue;
        const LoopVar& v = var(c.first);
        int pos = 0;
        for (size_t i = 0; i < st_.vars.size(); ++i) {
          if (st_.vars[i].name == v.name) pos = static_cast<int>(i);
        }
        const bool kernelLevel = !v.reduction && pos < kc_.k.sharedDepth;
        const int64_t span = kernelLevel ? v.tile : v.extent;
        int64_t base = v.min;
        if (c.second < 0) base += span - 1;
        low.constant += c.second * base;
        if (kernelLevel && v.numTiles > 1) low.coef["t_" + v.name] += c.second * v.tile;
        ext += std::abs(c.second) * (span - 1);
      }
      box.low.push_back(low);
      box.extents.push_back(ext);
    }
    box.valid = true;
    return box;
  }
  IterationBox writeBox() const {
    std::vector<Affine> subs;
    for (const auto& e : st_.lhsSubs) subs.push_back(ir::toAffine(e));
    return iterationBox({subs});
  }
  // every load of `tensor` in the stage; invalid when one of them is not affine
  IterationBox readBox(const std::string& tensor) const {
    std::vector<std::vector<Affine>> accesses;
    for (const auto& stmt : st_.stmts) {
      visit(stmt.rhs, [&](const ExprRef& e) {
        if (e->kind != Expr::Load || e->name != tensor) return;
        std::vector<Affine> subs;
        for (const auto& a : e->args) subs.push_back(ir::toAffine(a));
        accesses.push_back(subs);
      });
    }
    return iterationBox(accesses);
  }
  static std::string tileAffineStr(const Affine& a) {
    std::ostringstream ss;
    ss << a.constant;
    for (const auto& c : a.coef) {
      if (c.second != 0) ss << (c.second < 0 ? " - " : " + ") << std::abs(c.second) << " * " << c.first;
    }
    return ss.str();
  }
  const KernelCtx::Forward* forwardOf(const std::string& tensor) const {
    auto it = kc_.forwards.find(tensor);
    return it == kc_.forwards.end() ? nullptr : &it->second;
  }
  std::string forwardIndex(const KernelCtx::Forward& f, const std::vector<ExprRef>& subs) {
    std::ostringstream ss;
    for (size_t j = 0; j < subs.size(); ++j) {
      if (j) ss << " + ";
      ss << "((" << affineStr(ir::toAffine(subs[j])) << ") - (" << f.lows[j] << "))";
      if (f.strides[j] != 1) ss << " * " << f.strides[j];
    }
    return ss.str();
  }

  // The stage's result when nothing later in this kernel reads it back: it is stored with
  // device-scope write-through (buffer stores with the sc1 bit).  A plain or non-temporal store
  // leaves the line dirty in the L2 of its XCD, and everything still dirty when the last wavefront
  // ends is written back before the kernel completes: a result of a few MB then adds its whole
  // write-back time to the kernel (12.8 MB: 2.4 us) instead of overlapping it with the computation.
  // Byte offsets of a buffer access are 32 bits wide, which bounds the tensors this applies to.
  bool streamedStore() const {
    if (st_.atomic) return false;
    if (!kc_.opts.useReadOnlyCacheValue || viewBytes(st_.tensor) >= (int64_t(1) << 31)) return false;
    if (forwardOf(st_.tensor) || kc_.registerForwards.count(st_.tensor)) return true; // the later stages read the copy
    for (size_t j = stageIdx_ + 1; j < kc_.k.stages.size(); ++j) {
      if (tensorsRead(kc_.k.stages[j]).count(st_.tensor)) return false;
    }
    return true;
  }
  static std::string bufferName(const std::string& tensor) { return "rs" + tensor + "_"; }

  std::string storeStmt(const std::string& cond, const std::string& value) {
    std::string index = flatIndex(st_.tensor, st_.lhsSubs, "");
    if (st_.atomic) {
      const ReduceOp op = st_.stmts[0].op;
      const std::string fn =
          op == ReduceOp::Plus ? "__tc::atomicAccumulate" : "__tc::atomicCombine<" + opStruct(op, accType_) + ">";
      return "if (" + cond + ") " + fn + "(&p" + st_.tensor + "[" + index + "], " + value + ");";
    }
    std::string store = streamedStore()
        ? "__tc::storeThrough(" + bufferName(st_.tensor) + ", " + index + ", " + value + ");"
        : "p" + st_.tensor + "[" + index + "] = " + value + ";";
    {
      auto rf = kc_.registerForwards.find(st_.tensor);
      if (rf != kc_.registerForwards.end() && rf->second.producer <= stageIdx_) {
        if (stageIdx_ < rf->second.lastWriter) return rf->second.name + " = " + value + ";";
        return rf->second.name + " = " + value + "; if (" + cond + ") " + store;
      }
    }
    const KernelCtx::Forward* f = forwardOf(st_.tensor);
    if (f && f->producer == stageIdx_) {
      return "if (" + cond + ") { " + store + " " + f->ldsName + "[" + forwardIndex(*f, st_.lhsSubs) + "] = " + value + "; }";
    }
    return "if (" + cond + ") " + store;
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
    {
      auto rf = kc_.registerForwards.find(e->name);
      if (rf != kc_.registerForwards.end() && rf->second.producer < stageIdx_) return rf->second.name;
    }
    if (const KernelCtx::Forward* f = forwardOf(e->name)) {
      if (f->producer < stageIdx_) return f->ldsName + "[" + forwardIndex(*f, e->args) + "]";
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
        // half has no math library of its own: evaluated in float, rounded once
        const bool half = e->type.isFloat() && e->type.bits == 16;
        const ScalarType argType = half ? ScalarType{ScalarType::Float, 32} : e->type;
        std::string s = e->name + "(";
        for (size_t i = 0; i < e->args.size(); ++i) {
          s += (i ? ", " : "") + castTo(e->args[i], argType, accRef);
        }
        return half ? "((_Float16)" + s + "))" : s + ")";
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
        if (e->name == "%" && mt.bits == 16) return "((_Float16)fmodf((float)" + a + ", (float)" + b + "))";
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
    std::vector<Affine> forms;
    for (size_t j = 0; j < subs.size(); ++j) forms.push_back(ir::toAffine(subs[j]));
    if (columnSums_) {
      Affine part;
      part.valid = true;
      bool ok = true;
      std::vector<Affine> rest = forms;
      for (size_t j = 0; j < subs.size(); ++j) {
        Affine probe;
        Affine copy = rest[j];
        takeColumnTerms(copy, 1, probe);
        if (!anyTerm(probe)) continue;
        ok &= p.steps[j] == 1; // (a stepped dimension divides the whole difference)
        takeColumnTerms(rest[j], p.ldsStrides[j], part);
      }
      if (ok && anyTerm(part)) {
        forms = rest;
        ss << columnSumOf(part) << " + ";
      }
    }
    for (size_t j = 0; j < subs.size(); ++j) {
      if (j) ss << " + ";
      ss << "((" << affineStr(forms[j]) << ") - lo" << stageIdx_ << "_" << p.tensor << "_" << j << ")";
      if (p.steps[j] != 1) ss << " / " << p.steps[j]; // exact: every access is a whole number of steps from the origin
      if (p.ldsStrides[j] != 1) ss << " * " << p.ldsStrides[j];
    }
    if (subs.empty()) ss << "0";
    if (p.buffers == 2 && !readBuffer_.empty()) ss << " + " << readBuffer_ << " * " << p.elems;
    return ss.str();
  }
  // Which of the two copies of a double-buffered array is read and which is written (expressions
  // with value 0 or 1; empty outside the software pipeline over the reduction tiles).
  std::string readBuffer_, writeBuffer_;

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
    // (with the reduction split over wavefronts a wavefront has one tile: nothing to keep)
    return MT <= 16 && BT == 1 && ceilDiv(KT, 4) <= kMaxResidentSteps && mfmaKSplit() == 1;
  }

  // Output tiles of 16x16 per block and reduction steps per lane of a matrix-core stage.
  void mfmaCounts(int64_t& tiles, int64_t& ksteps) const {
    int64_t MT = 1, NT = 1, BT = 1, KT = 1;
    for (const auto& n : st_.mfmaM) MT *= var(n).tile;
    for (const auto& n : st_.mfmaN) NT *= var(n).tile;
    for (const auto& n : st_.mfmaBatch) BT *= var(n).tile;
    for (const auto& n : st_.mfmaK) KT *= var(n).tile;
    tiles = BT * ceilDiv(MT, 16) * ceilDiv(NT, 16);
    ksteps = ceilDiv(KT, 4);
  }
  // Reduction split over wavefronts.  A block with fewer output tiles than wavefronts would leave
  // wavefronts idle while the busy ones walk the whole reduction: the steps of a tile are divided
  // evenly among `split` wavefronts instead, whose partial tiles meet in LDS (one 16-byte write per
  // lane, a barrier, the owner of the tile adds them up).  1: no split.
  static constexpr int64_t kMinStepsPerSplit = 8;
  int64_t mfmaKSplit() const {
    if (!st_.mfma || !kSplitAllowed_) return 1;
    int64_t tiles, ksteps;
    mfmaCounts(tiles, ksteps);
    if (tiles >= st_.waves) return 1;
    int64_t split = std::min(st_.waves / tiles, ksteps / kMinStepsPerSplit);
    if (split < 2) return 1;
    // the fewest wavefronts that keep the steps of the busiest one at that minimum
    return ceilDiv(ksteps, ceilDiv(ksteps, split));
  }
  int64_t mfmaKSplitBytes() const {
    int64_t tiles, ksteps;
    mfmaCounts(tiles, ksteps);
    return (mfmaKSplit() - 1) * tiles * 64 * 16;
  }
  std::string kSplitName() const { return "ksplit" + std::to_string(stageIdx_) + "_"; }

  bool fullRegisterTile() const {
    for (const auto& v : st_.vars) {
      if (!st_.mfma && !v.reduction && !v.unrolled && v.perThread > 1) return false;
    }
    return true;
  }

  void planPromotions(const StageStmt& s, int64_t& ldsBudgetBytes) {
    if (!kc_.opts.useSharedMemoryValue) return;
    if (s.redVars.empty() && st_.mfma) return;
    bool reductionTiled = false;
    for (const auto& r : s.redVars) reductionTiled |= var(r).numTiles > 1;
    bool inside = reductionTiled &&
        (!kc_.opts.hasSharedDepth || kc_.opts.sharedDepthValue > static_cast<uint32_t>(st_.numParallel));
    // Per-thread loops that stay loops enclose the whole statement, the reduction tile loop
    // included: a copy per reduction tile would be repeated by every one of their iterations.
    // Footprints of the whole block tile are staged once, in front of those loops.
    if (inside && !fullRegisterTile()) return;
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
    // (An M-side operand that the wavefronts keep in registers is staged as well: every wavefront
    // of the block needs all of it, a lane's share is one row, so reading it straight from global
    // memory costs one cache line per lane and load where the cooperative copy moves whole lines.)
    for (const auto& acc : accesses) {
      if (bad.count(acc.first)) continue;
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
        int64_t step = 0; // gcd of everything that moves an access along this dimension
        for (const auto& cv : ref[j].coef) {
          const int64_t span = spanOf(var(cv.first), inside);
          ext += std::abs(cv.second) * (span - 1);
          if (span > 1) step = gcd(step, cv.second);
        }
        for (const auto& a : acc.second) step = gcd(step, a[j].constant - lo);
        if (step > 1) ext = (ext - 1) / step + 1;
        c.fp.minConst.push_back(lo);
        c.p.extents.push_back(ext);
        c.p.steps.push_back(std::max<int64_t>(1, step));
        elems *= ext;
      }
      c.p.reuse = static_cast<int64_t>(iterations * acc.second.size() / static_cast<double>(elems));
      // Worth a copy when elements are used more than once, or when the threads of a wavefront
      // walk a slower dimension of the tensor while the cooperative copy reads whole rows
      // (promotionImprovesCoalescing, tc/core/polyhedral/cuda/memory_promotion_heuristic.cc:211-244).
      const bool coalesces = lanesWalkOuterDim(ref) && c.p.extents.back() >= 8;
      if (c.p.reuse < 2 && !coalesces) continue;
      // A footprint of fewer elements than the block has threads is read where it lies: the copy
      // would put two block barriers around less than one load per thread (the 16x16 factors of
      // the Kronecker product, staged inside its tile loops, cost 3 us of 17).
      if (elems < kc_.NT()) continue;
      // Pitches.  pad[j] = elements added to the distance between consecutive indices of dimension j.
      const size_t nd = ref.size();
      std::vector<int64_t> pad(nd, 0);
      auto stridesWith = [&](const std::vector<int64_t>& pd) {
        std::vector<int64_t> str(nd, 1);
        for (size_t j = nd - 1; j-- > 0;) str[j] = str[j + 1] * c.p.extents[j + 1] + pd[j];
        return str;
      };
      // lanes that walk a slower dimension: an odd row length spreads them over the banks
      if (nd >= 2 && c.p.extents.back() > 1 && c.p.extents.back() % 2 == 0 && lanesWalkOuterDim(ref)) pad[nd - 2] += 1;
      if (st_.mfma && nd >= 2 && kMfmaPad > 0) {
        const bool isA = acc.first == contractionOperand(s.rhs->args[st_.mfmaSwapOperands ? 1 : 0])->name;
        // The 16 lanes of a group walk the M- (or N-) side variable.  When that variable is not in
        // the last subscript, consecutive lanes are a whole pitch apart and a pitch that is a
        // multiple of 8 elements piles them onto few LDS banks: four elements of padding spread 16
        // rows over 8 bank groups while rows stay 16-byte aligned for the copies.
        const auto& side = isA ? st_.mfmaM : st_.mfmaN;
        int sideDim = -1;
        for (size_t j = 0; j < nd; ++j) {
          for (const auto& n : side) {
            if (ref[j].coefOf(n) != 0) sideDim = static_cast<int>(j);
          }
        }
        if (sideDim >= 0 && sideDim + 1 < static_cast<int>(nd) && stridesWith(pad)[sideDim] % 8 == 0) pad[sideDim] += kMfmaPad;
        // The four lane groups of a wavefront own consecutive quarters of the flattened reduction:
        // at every step their addresses differ by the same number of elements, and when that is a
        // multiple of the 32 banks the groups of each half of the wavefront collide.  Padding the
        // pitch of the outermost reduction variable's dimension moves the groups apart.
        int64_t KT = 1, innerProd = 1;
        for (size_t i = 0; i < st_.mfmaK.size(); ++i) {
          int64_t t = spanOf(var(st_.mfmaK[i]), inside);
          KT *= t;
          if (i > 0) innerProd *= t;
        }
        const int64_t quarter = ceilDiv(KT, 4);
        int kDim = -1;
        for (size_t j = 0; j < nd; ++j) {
          if (ref[j].coefOf(st_.mfmaK[0]) != 0) kDim = static_cast<int>(j);
        }
        if (quarter % innerProd == 0 && kDim >= 0 && kDim + 1 < static_cast<int>(nd)) {
          auto groupStride = [&](const std::vector<int64_t>& pd) {
            auto str = stridesWith(pd);
            int64_t g = 0;
            for (size_t j = 0; j < nd; ++j) g += ref[j].coefOf(st_.mfmaK[0]) * str[j];
            return g * (quarter / innerProd);
          };
          if (groupStride(pad) % 32 == 0) {
            for (int64_t extra = kMfmaPad; extra <= 3 * kMfmaPad; extra += kMfmaPad) {
              std::vector<int64_t> trial = pad;
              trial[kDim] += extra;
              if (groupStride(trial) % 32 != 0) {
                pad = trial;
                break;
              }
            }
          }
        }
      }
      c.p.ldsStrides = stridesWith(pad);
      c.p.elems = nd == 0 ? 1 : c.p.ldsStrides[0] * c.p.extents[0];
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
    // Two copies of the arrays staged per reduction tile when the matrix-core software pipeline
    // will run over them and LDS has the room.
    if (st_.mfma && kc_.opts.prefetchSharedValue) {
      int64_t extra = 0, stagingRegs = 0;
      bool any = false;
      for (const auto& p : st_.promotions) {
        if (!p.insideReductionTiles) continue;
        any = true;
        extra += p.elems * st_.views.at(p.tensor).type.bytes();
        stagingRegs += copyRegisters(p);
      }
      // (the pipeline's own conditions, emitMfma: staged per reduction tile, at most 64 staging registers)
      if (any && stagingRegs <= 64 && extra <= ldsBudgetBytes) {
        ldsBudgetBytes -= extra;
        for (auto& p : st_.promotions) {
          if (p.insideReductionTiles) p.buffers = 2;
        }
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
    if (mfmaKSplit() > 1) {
      em_.line("__shared__ __attribute__((aligned(16))) float " + kSplitName() + "[" + std::to_string(mfmaKSplitBytes() / 4) + "];");
    }
    for (const auto& p : st_.promotions) {
      if (p.sharedWithEarlierStage) continue;
      em_.line("__shared__ __attribute__((aligned(16))) " + st_.views.at(p.tensor).type.cName() + " " + p.ldsName +
               "[" + std::to_string(p.elems * p.buffers) + "];");
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
    int64_t step; // tensor elements between neighbouring footprint elements
    std::string lo;
    int64_t loGcd; // every value of `lo` is a multiple of this (0: lo is always 0)
    bool inside;   // the footprint never leaves the tensor in this dimension: no bounds test
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

  // Whether the footprint stays inside the tensor in view dimension j for every tile: the lowest
  // and highest values footprintLow(p, j) can take, from the same terms.
  bool footprintAlwaysInside(const Promotion& p, size_t j) const {
    const Footprint& fp = footprints_.at(p.tensor);
    int64_t lo = fp.minConst[j], hi = fp.minConst[j];
    for (const auto& c : fp.coefs[j].coef) {
      const LoopVar& v = var(c.first);
      bool fixed = (v.reduction && !p.insideReductionTiles) || v.numTiles == 1;
      int64_t vlo = v.min, vhi = fixed ? v.min : v.min + (v.numTiles - 1) * v.tile;
      if (c.second < 0) {
        vlo += spanOf(v, p.insideReductionTiles) - 1;
        vhi += spanOf(v, p.insideReductionTiles) - 1;
      }
      int64_t a = c.second * vlo, b = c.second * vhi;
      lo += std::min(a, b);
      hi += std::max(a, b);
    }
    return lo >= 0 && hi + (p.extents[j] - 1) * p.steps[j] + 1 <= st_.views.at(p.tensor).extents[j];
  }

  CopyPlan copyPlan(const Promotion& p) const {
    const TensorView& view = st_.views.at(p.tensor);
    auto gStridesFull = makeStridesFromSizes(view.extents);
    CopyPlan plan;
    for (auto e : p.extents) plan.count *= e;
    for (size_t j = 0; j < p.extents.size(); ++j) {
      plan.dims.push_back(CopyDim{p.extents[j], view.extents[j], gStridesFull[j], p.ldsStrides[j], p.steps[j],
                                  loPrefix(p) + std::to_string(j), footprintLowGcd(p, j), footprintAlwaysInside(p, j)});
    }
    auto& dims = plan.dims;
    while (dims.size() >= 2) {
      CopyDim& in = dims.back();
      CopyDim& out = dims[dims.size() - 2];
      bool full = in.extent == in.tensorExtent && in.step == 1 && out.step == 1 && out.lStride == in.lStride * in.extent &&
          out.gStride == in.gStride * in.tensorExtent;
      if (!full) break;
      // (out, in) -> one dimension of extent out*in starting at out.lo * in.extent (in.lo is 0)
      out.lo = "(" + out.lo + ") * " + std::to_string(in.extent);
      out.loGcd *= in.extent;
      out.inside = out.inside && in.inside;
      out.extent *= in.extent;
      out.tensorExtent *= in.tensorExtent;
      out.gStride = in.gStride;
      out.lStride = in.lStride;
      dims.pop_back();
    }
    plan.elemType = view.type.cName();
    plan.regType = plan.elemType;
    // (groups of four elements: 16 bytes of floats, 8 bytes of halves)
    if (view.type.isFloat() && (view.type.bits == 32 || view.type.bits == 16) && !dims.empty()) {
      const CopyDim& in = dims.back();
      bool ok = in.gStride == 1 && in.lStride == 1 && in.step == 1 && in.extent % 4 == 0 && in.tensorExtent % 4 == 0 &&
          in.loGcd % 4 == 0;
      for (size_t j = 0; j + 1 < dims.size(); ++j) ok &= dims[j].gStride % 4 == 0 && dims[j].lStride % 4 == 0;
      if (ok) {
        plan.vec = 4;
        plan.regType = view.type.bits == 32 ? "__tc::floatx4" : "__tc::halfx4";
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
  // `loopIters`: iterations the enclosing loops run in total (a chunked loop may overshoot
  // plan.iters).
  void emitCopyStep(const Promotion& p, const CopyPlan& plan, const std::string& itExpr, const std::string& regs,
                    const std::string& slot, bool loads, int64_t loopIters) {
    const auto& dims = plan.dims;
    std::string unit = "(" + itExpr + ") * " + std::to_string(kc_.NT()) + " + tid_";
    em_.line("const int c_ = " + (plan.vec > 1 ? std::to_string(plan.vec) + " * (" + unit + ")" : unit) + ";");
    // Only the last iterations can reach past the end of the footprint, and only when the
    // footprint is not a whole number of the steps the loops make: the test names the iteration, so it
    // folds away in the unrolled copies of the others.  Threads past the end skip their access
    // (whole wavefronts of them skip the instruction).
    const int64_t perIter = kc_.NT() * plan.vec;
    const int64_t fullIters = plan.count / perIter;
    const bool ragged = loopIters * perIter > plan.count;
    const std::string live = ragged ? "(" + itExpr + ") < " + std::to_string(fullIters) + " || c_ < " + std::to_string(plan.count) : "";
    int64_t div = plan.count;
    std::string cond, gidx, lidx;
    bool outermost = true; // the first dimension with more than one element needs no wrap-around
    for (size_t j = 0; j < dims.size(); ++j) {
      div /= dims[j].extent;
      std::string l = "l" + std::to_string(j) + "_";
      if (dims[j].extent == 1) {
        em_.line("const int " + l + " = 0;");
      } else {
        std::string e = "c_";
        if (div > 1) e = "(" + e + " / " + std::to_string(div) + ")";
        if (!outermost) e = e + " % " + std::to_string(dims[j].extent);
        outermost = false;
        em_.line("const int " + l + " = " + e + ";");
      }
      if (loads) {
        std::string g = "g" + std::to_string(j) + "_";
        em_.line("const int " + g + " = " + dims[j].lo + " + " + l + (dims[j].step != 1 ? " * " + std::to_string(dims[j].step) : "") + ";");
        if (!dims[j].inside) {
          cond += (cond.empty() ? "" : " && ") + std::string("(unsigned)") + g + " < " + std::to_string(dims[j].tensorExtent) + "u";
        }
        gidx += (j ? " + " : "") + std::string(kc_.wide ? "(int64)" : "") + g +
            (dims[j].gStride != 1 ? " * " + std::to_string(dims[j].gStride) : "");
      }
      lidx += (j ? " + " : "") + l + (dims[j].lStride != 1 ? " * " + std::to_string(dims[j].lStride) : "");
    }
    if (dims.empty()) gidx = lidx = "0";
    std::string cast = plan.vec > 1 ? "*(const " + plan.regType + "u*)&" : "";
    std::string lcast = plan.vec > 1 ? "*(" + plan.regType + "*)&" : "";
    std::string guard = live.empty() ? "" : "if (" + live + ") ";
    if (loads) {
      // inside the footprint but outside the tensor (halo of a partial tile): a clamped address,
      // so that the loads stay unconditional and issue back to back; the value is never used
      std::string addr = cond.empty() ? gidx : "(" + cond + ") ? (" + gidx + ") : 0";
      em_.line(guard + regs + "[" + slot + "] = " + cast + "p" + p.tensor + "[" + addr + "];");
    } else {
      if (p.buffers == 2 && !writeBuffer_.empty()) lidx += " + " + writeBuffer_ + " * " + std::to_string(p.elems);
      em_.line(guard + lcast + p.ldsName + "[" + lidx + "] = " + regs + "[" + slot + "];");
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
    emitCopyStep(p, plan, "it_", regs, "it_", loads, plan.iters);
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
      emitCopyStep(p, plan, base + "it_", "stage_", "it_", loads, ceilDiv(plan.iters, chunk) * chunk);
      em_.close();
    }
    em_.close();
  }

  // Stages several footprints at once: the global loads of all of them are issued before the
  // first LDS store, so that their latencies overlap, when a thread's share fits in registers.
  void emitCopyInGroup(const std::vector<const Promotion*>& ps) {
    int64_t regs = 0;
    for (const auto* p : ps) regs += copyRegisters(*p);
    if (ps.size() < 2 || regs > (kc_.opts.unrollCopySharedValue ? 64 : 32)) {
      for (const auto* p : ps) emitCopyIn(*p);
      return;
    }
    for (const auto* p : ps) declareLows(*p);
    em_.open("");
    for (const auto* p : ps) em_.line(copyRegisterDecl(*p, "stage_" + p->tensor + "_"));
    for (const auto* p : ps) emitCopyLoads(*p, "stage_" + p->tensor + "_");
    for (const auto* p : ps) emitCopyStores(*p, "stage_" + p->tensor + "_");
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
    const bool staged = &s == promotedPointwise_;
    if (staged) {
      em_.open("");
      if (stagedAheadOfPointLoops_) {
        for (const auto& p : st_.promotions) activePromotions_.insert(p.tensor);
      } else {
        stageOutsideFootprints();
      }
    }
    emitPointwiseBody(s);
    if (staged) {
      for (const auto& p : st_.promotions) activePromotions_.erase(p.tensor);
      em_.close();
    }
  }

  // Copies the stage's footprints of one kind (inside / outside the reduction tile loop) into LDS,
  // between two barriers, and makes the statement's loads read them; footprints an earlier stage
  // has staged are only addressed.  The barrier in front protects the readers of what the arrays
  // held before: there are none ahead of the first copy of the first stage of a kernel without
  // kernel-level loops.
  void stageFootprints(bool inside) {
    std::vector<const Promotion*> group;
    for (const auto& p : st_.promotions) {
      if (p.insideReductionTiles != inside) continue;
      activePromotions_.insert(p.tensor);
      if (p.sharedWithEarlierStage) {
        declareLows(p);
      } else {
        group.push_back(&p);
      }
    }
    if (group.empty()) return;
    if (inside || stageIdx_ > 0 || kc_.kernelLoops || stageTileLoops_ || copiedBefore_) em_.line("__syncthreads();");
    copiedBefore_ = true;
    emitCopyInGroup(group);
    em_.line("__syncthreads();");
  }
  void stageOutsideFootprints() { stageFootprints(false); }

  void emitPointwiseBody(const StageStmt& s) {
    int n = openUnrolled();
    inCachedReduction_ = cachedPointwise_;
    cacheSlot_ = "a_";
    em_.line("acc_[a_] = " + castTo(s.rhs, accType_, accValid_ ? "acc_[a_]" : "") + ";");
    inCachedReduction_ = false;
    closeN(n);
  }

  void preloadAcc() {
    int n = openUnrolled();
    auto rf = kc_.registerForwards.find(st_.tensor);
    if (rf != kc_.registerForwards.end() && rf->second.producer < stageIdx_) {
      em_.line("acc_[a_] = " + rf->second.name + ";");
    } else {
      em_.line("acc_[a_] = p" + st_.tensor + "[" + flatIndex(st_.tensor, st_.lhsSubs, "") + "];");
    }
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
      if (stagedAheadOfPointLoops_ && !inside) {
        for (const auto& p : st_.promotions) activePromotions_.insert(p.tensor);
        return;
      }
      if (suppressCopy && !inside) {
        for (const auto& p : st_.promotions) {
          if (!p.insideReductionTiles) {
            declareLows(p);
            activePromotions_.insert(p.tensor);
          }
        }
        return;
      }
      stageFootprints(inside);
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
        // A double-precision value combined under a condition: hipcc (ROCm 7.0 and 7.2, -O1 and
        // up) does not finish compiling `r = tanh(x); if (c) acc = max(acc, r)` inside these loops;
        // with the value pinned in a register first it compiles in a second.  Every conditional
        // combine in double precision is pinned, whatever computes the value: the JIT has no
        // time limit, a second trigger of the defect would block compile() for good.
        if (accType_.isFloat() && accType_.bits == 64) {
          em_.line(accType_.cName() + " r_ = " + rhs + ";");
          em_.line("asm volatile(\"\" : \"+v\"(r_));");
        } else {
          em_.line("const " + accType_.cName() + " r_ = " + rhs + ";");
        }
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
  // Footprints are planned for the stage's reduction statement; a stage without one (a stencil,
  // say: several accesses per element through overlapping windows) plans them for its first
  // statement that loads anything.
  void plan(int64_t& ldsBudgetBytes) {
    if (mfmaKSplit() > 1) {
      if (mfmaKSplitBytes() > ldsBudgetBytes) {
        kSplitAllowed_ = false;
      } else {
        ldsBudgetBytes -= mfmaKSplitBytes();
      }
    }
    for (const auto& s : st_.stmts) {
      if (!s.redVars.empty()) {
        planPromotions(s, ldsBudgetBytes);
        return;
      }
    }
    for (const auto& s : st_.stmts) {
      bool loads = false;
      visit(s.rhs, [&](const ExprRef& e) { loads |= e->kind == Expr::Load && e->name != st_.tensor; });
      if (loads) {
        planPromotions(s, ldsBudgetBytes);
        promotedPointwise_ = st_.promotions.empty() ? nullptr : &s;
        return;
      }
    }
  }

  // The footprint origins of promotion `p` as text, for comparing the footprints of two stages.
  std::string footprintKey(const Promotion& p) const {
    std::ostringstream ss;
    ss << p.tensor << (p.insideReductionTiles ? "|inside" : "|outside");
    for (size_t j = 0; j < p.extents.size(); ++j) {
      ss << "|" << p.extents[j] << ":" << p.steps[j] << ":" << p.ldsStrides[j] << ":" << footprintLow(p, j);
    }
    return ss.str();
  }
  // Whether every footprint origin is fixed by the block ids and the kernel-level tile loops: the
  // staged data then stays valid from one stage of a kernel-level iteration to the next.
  bool footprintFixedPerKernelIteration(const Promotion& p) const {
    if (p.insideReductionTiles) return false;
    const Footprint& fp = footprints_.at(p.tensor);
    for (const auto& dim : fp.coefs) {
      for (const auto& c : dim.coef) {
        if (c.second == 0) continue;
        const LoopVar& v = var(c.first);
        if (v.reduction || v.numTiles == 1) continue;
        bool kernelLevel = false;
        for (int i = 0; i < kc_.k.sharedDepth && i < st_.numParallel; ++i) kernelLevel |= st_.vars[i].name == v.name;
        if (!kernelLevel) return false;
      }
    }
    return true;
  }
  std::vector<Promotion>& mutablePromotions() { return st_.promotions; }

  // Declares i_<v> (and p_<v>) for every variable of `group` from the flattened position `pos`
  // inside the block tile (row-major over the group's tile extents, last variable fastest) and
  // returns the predicate "position exists".
  // (inRange: the caller knows the position to lie inside the group's tile box; no test, and no
  // clamp that would keep the compiler from folding the decoded indices into address immediates)
  std::string decodeGroup(const std::vector<std::string>& group, const std::string& pos, bool clamp = false,
                          bool inRange = false) {
    int64_t total = 1;
    for (const auto& n : group) total *= var(n).tile;
    std::string pred = inRange ? std::string("true") : pos + " < " + std::to_string(total);
    // clamped: positions past the end alias the last valid one, so that addresses computed from
    // the decoded indices are always legal (used for operands whose surplus lanes are discarded)
    std::string src = pos;
    if (clamp && !inRange) {
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
    // (a float16 operand is read as it is and converted where its value enters a float register)
    const ExprRef loadA = contractionOperand(s.rhs->args[st_.mfmaSwapOperands ? 1 : 0]); // holds the M-side variables
    const ExprRef loadB = contractionOperand(s.rhs->args[st_.mfmaSwapOperands ? 0 : 1]); // holds the N-side variables
    em_.line("// matrix cores: " + std::to_string(tiles) + " tiles of 16x16 per block, " + std::to_string(ksteps) +
             " steps of v_mfma_f32_16x16x4_f32 each, " + std::to_string(st_.waves) + " wavefront(s)");
    // (the register-resident operand is requested first: its latency overlaps the LDS staging)
    // Wavefronts that still fetch and stage their operands go ahead of the ones that already
    // multiply: all blocks of a compute unit start together, the first whose operands arrive fill
    // the matrix pipeline, and at equal priority the instructions of the others (waits, LDS
    // stores, the barrier) were issued so rarely that the last block of a compute unit began to
    // multiply 4 us after the first (per-wavefront timestamps on the 16-channel group convolution).
    bool stagesOutside = false;
    for (const auto& p : st_.promotions) stagesOutside |= !p.insideReductionTiles && !p.sharedWithEarlierStage;
    const bool raisePriority = stagesOutside && !suppressCopy;
    if (raisePriority) em_.line("__builtin_amdgcn_s_setprio(3);");
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
    const int64_t split = mfmaKSplit();
    const int64_t stepsPerWave = ceilDiv(ksteps, split);
    const bool unevenSplit = stepsPerWave * split != ksteps; // the last slice has surplus steps
    const std::string kx = split > 1 ? "kq_" : "ks_"; // counter of a wavefront's own steps
    // Opens the loop over the reduction steps of a lane, decodes the reduction indices of the
    // step and declares kok_ when surplus steps exist; returns whether it did.
    // Decodes the reduction indices of step ks_ and declares kok_ when surplus steps exist;
    // returns whether it did.
    auto declareStepIndices = [&]() {
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
    auto openSteps = [&](int64_t count, int64_t first = 0, int64_t last = -1) {
      em_.line(count <= 128 ? "#pragma unroll" : "#pragma unroll 4");
      if (split > 1) {
        // slice sl_ of the steps: ks_ is the step within the whole reduction
        em_.open("for (int kq_ = " + std::to_string(first) + "; kq_ < " + std::to_string(last < 0 ? count : last) + "; ++kq_)");
        em_.line("const int ks_ = sl_ * " + std::to_string(stepsPerWave) + " + kq_;");
      } else {
        em_.open("for (int ks_ = " + std::to_string(first) + "; ks_ < " + std::to_string(last < 0 ? ksteps : last) + "; ++ks_)");
      }
      return declareStepIndices();
    };
    // An operand read straight from global memory whose elements of consecutive steps of a lane
    // are consecutive in memory (the reduction subscripts are jointly contiguous): four steps
    // can then be fetched with one 16-byte load.
    auto contiguousAlongSteps = [&](const ExprRef& load) {
      if (!aligned || quarter * 4 != KT || activePromotions_.count(load->name) || forwardOf(load->name)) return false;
      if (st_.views.at(load->name).type.bits != 32) return false;
      Affine fa = flatAffine(load->name, load->args);
      if (!fa.valid) return false;
      int64_t expect = 1;
      for (size_t i = st_.mfmaK.size(); i-- > 0;) {
        const LoopVar& v = var(st_.mfmaK[i]);
        if (fa.coefOf(v.name) != expect) return false;
        expect *= v.tile;
      }
      return true;
    };
    // surplus reduction steps must contribute exact zeros
    auto operandValue = [&](const ExprRef& load, bool masked) {
      std::string text = loadStr(load, "");
      return masked ? "(kok_ ? " + text + " : 0.0f)" : text;
    };
    const bool resident = mfmaKeepsMOperandInRegisters();
    bool residentFromLds = false;
    for (const auto& p : st_.promotions) residentFromLds |= resident && p.tensor == loadA->name;
    if (resident) em_.line("float am_[" + std::to_string(ksteps) + "];");
    // fills am_: a lane's M-side operand values, one per reduction step
    auto fillResident = [&]() {
      em_.open("");
      em_.line("const int mt_ = 0, bt_ = 0;");
      em_.line("(void)mt_; (void)bt_;");
      if (!st_.mfmaBatch.empty()) decodeGroup(st_.mfmaBatch, "bt_", true, true);
      em_.line("const int mposa_ = lm_;");
      decodeGroup(st_.mfmaM, "mposa_", true, MT % 16 == 0);
      // consecutive steps of a lane read consecutive elements when the operand's reduction
      // subscripts are jointly contiguous: four steps are then fetched with one 16-byte load
      bool contiguous = !residentFromLds && !forwardOf(loadA->name) && aligned && quarter * 4 == KT && ksteps % 4 == 0 &&
          st_.views.at(loadA->name).type.bits == 32;
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
        bool masked = openSteps(ksteps);
        em_.line("am_[ks_] = " + operandValue(loadA, masked) + ";");
        em_.close();
      }
      em_.close();
    };
    if (resident && !residentFromLds) fillResident();
    // Epilogue operands that do not depend on the column (a bias per output row, say) are the
    // same for every tile of the wavefront: fetched once, ahead of the tile loop.
    hoistedLoads_.clear();
    size_t hoistedCount = 0;
    std::vector<std::string> hoistedTexts, hoistedTypes;
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
        if (!st_.mfmaBatch.empty()) decodeGroup(st_.mfmaBatch, "bt_", true, true);
        decodeGroup(st_.mfmaM, "mpos_", true, MT % 16 == 0);
        for (size_t h = 0; h < invariant.size(); ++h) {
          em_.line("eh" + std::to_string(h) + "_[r_] = " + invariant[h].first + ";");
        }
        em_.close();
        for (size_t h = 0; h < invariant.size(); ++h) {
          hoistedLoads_[invariant[h].first] = "eh" + std::to_string(h) + "_[r_]";
        }
        hoistedCount = invariant.size();
        hoistedTexts.clear();
        for (const auto& h : invariant) hoistedTexts.push_back(h.first);
        hoistedTypes.clear();
        for (const auto& h : invariant) hoistedTypes.push_back(st_.views.at(h.second->name).type.cName());
      }
    }
    // Reduction tiling: the outermost reduction variable may run over several tiles; operands
    // staged per reduction tile are copied inside that loop and the accumulators of all output
    // tiles of a wavefront live in registers across it.
    const LoopVar& k0 = var(st_.mfmaK[0]);
    const bool kTiled = k0.numTiles > 1;
    // Surplus columns.  When the columns of a block tile are not a multiple of 16, the last column
    // tile of every row tile is mostly padding (196 pixels = 12 tiles + 4 columns).  Up to twelve
    // surplus columns go through v_mfma_f32_4x4x1_16B_f32 instead, four columns a pass: its 16
    // blocks are the 4 row quads of the row tile x the 4 quarters of the reduction, so a lane
    // multiplies the same M-side value as in the 16x16x4 instruction (row lm_, quarter lj_) with
    // the N-side value of column (lane & 3), and the four partial sums of an output element sit
    // in the lanes that differ in bits 4 and 5.  A pass costs a quarter of a full tile.
    const int64_t remCols = NT % 16;
    const int64_t remPasses = ceilDiv(remCols, 4);
    bool quarterTiles = !kTiled && split == 1 && remCols != 0 && remPasses <= 3 && s.init &&
                        stepsPerWave <= kMaxResidentSteps;
    if (quarterTiles) {
      // Only where the busiest wavefront gets less to do: units are dealt round-robin, full tiles
      // first, and a pass is priced at half a tile (a quarter of the multiplications, all of the
      // operand reads, an exchange between lanes).
      const int64_t full = BT * numMT * (NT / 16), passes = BT * numMT * remPasses, W = st_.waves;
      double busiest = 0;
      for (int64_t w = 0; w < W; ++w) {
        double cost = 0;
        for (int64_t u = w; u < full + passes; u += W) cost += u < full ? 1.0 : 0.5;
        busiest = std::max(busiest, cost);
      }
      quarterTiles = busiest < static_cast<double>(ceilDiv(tiles, W));
    }
    const int64_t numNTfull = quarterTiles ? NT / 16 : numNT;
    const int64_t fullTiles = BT * numMT * numNTfull;
    const int64_t remUnits = quarterTiles ? BT * numMT * remPasses : 0;
    const int64_t tilesPerWave = ceilDiv(quarterTiles ? fullTiles + remUnits : tiles, st_.waves);
    // (in a quarter-tile pass lane l finishes rows 4*((l >> 2) & 3) .. +3 of column (l & 3))
    const std::string quadOfLane = "((threadIdx.x >> 2) & 3)";
    if (quarterTiles && hoistedCount > 0) {
      for (size_t h = 0; h < hoistedCount; ++h) em_.line(hoistedTypes[h] + " er" + std::to_string(h) + "_[4];");
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int bt_ = 0, mpos_ = 4 * " + quadOfLane + " + r_;");
      em_.line("(void)bt_;");
      if (!st_.mfmaBatch.empty()) decodeGroup(st_.mfmaBatch, "bt_", true, true);
      decodeGroup(st_.mfmaM, "mpos_", true, MT % 16 == 0);
      for (size_t h = 0; h < hoistedCount; ++h) em_.line("er" + std::to_string(h) + "_[r_] = " + hoistedTexts[h] + ";");
      em_.close();
    }
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
      stageFootprints(inside);
    };
    // decodes the output tile tl_ of this wavefront: batch and column indices, nok_
    // (columnsCached: the column indices of the unrolled tile j_ were decoded ahead of the staging)
    bool columnsCached = false;
    auto cachedColumns = [&]() {
      for (size_t i = 0; i < st_.mfmaN.size(); ++i) {
        em_.line("const int " + iv(var(st_.mfmaN[i])) + " = dn" + std::to_string(i) + "_[j_];");
        em_.line("(void)" + iv(var(st_.mfmaN[i])) + ";");
      }
      em_.line("const bool nok_ = dok_[j_];");
      em_.line("(void)nok_;");
    };
    auto decodeTile = [&]() {
      em_.line("const int nt_ = tl_ % " + std::to_string(numNTfull) + ", mt_ = (tl_ / " + std::to_string(numNTfull) + ") % " +
               std::to_string(numMT) + ", bt_ = tl_ / " + std::to_string(numNTfull * numMT) + ";");
      em_.line("(void)nt_;");
      // A row of the product depends on one row of the M-side operand only and a column on one
      // column of the N-side operand, so lanes past the end of a partial tile may load any legal
      // element (clamped indices): their results are never stored.
      std::string bok = st_.mfmaBatch.empty() ? "true" : decodeGroup(st_.mfmaBatch, "bt_", true, true);
      em_.line("const bool bok_ = " + bok + ";");
      if (columnsCached) {
        cachedColumns();
        return;
      }
      em_.line("const int npos_ = nt_ * 16 + lm_;");
      em_.line("const bool nok_ = bok_ && " + decodeGroup(st_.mfmaN, "npos_", true, quarterTiles || NT % 16 == 0) + ";");
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
      em_.line("const bool moka_ = bok_ && " + decodeGroup(st_.mfmaM, "mposa_", true, MT % 16 == 0) + ";");
      em_.line("(void)moka_;");
      // `count` steps of this wavefront
      auto steps = [&](int64_t count) {
        if (count <= kMaxResidentSteps) {
          // The operand values of all steps first, then the chain of multiplications: every read is
          // in flight before the first result is needed, and the multiplications wait for nothing
          // but their own operands (10.5 -> 10.0 us on the 16-channel 3x3 group convolution).
          em_.line("float bq_[" + std::to_string(count) + "];");
          if (!resident) em_.line("float aq_[" + std::to_string(count) + "];");
          // operands whose steps are consecutive in memory: 16-byte loads for groups of four
          // steps, single loads for the rest (a lane of the 128x1000x1024 matmul fetches its 63
          // values of the first operand with 15 + 3 loads instead of 63, each of which touched
          // 64 cache lines per wavefront)
          auto vectorLoads = [&](const ExprRef& load, const std::string& regs) {
            const int64_t groups = count / 4;
            em_.line("#pragma unroll");
            em_.open("for (int kv_ = 0; kv_ < " + std::to_string(groups) + "; ++kv_)");
            if (split > 1) {
              em_.line("const int kq_ = 4 * kv_;");
              em_.line("const int ks_ = sl_ * " + std::to_string(stepsPerWave) + " + kq_;");
            } else {
              em_.line("const int ks_ = 4 * kv_;");
            }
            declareStepIndices();
            em_.line("const __tc::floatx4 v_ = *(const __tc::floatx4u*)&p" + load->name + "[" + flatIndex(load->name, load->args, "") + "];");
            em_.line(regs + "[" + kx + "] = v_[0]; " + regs + "[" + kx + " + 1] = v_[1]; " + regs + "[" + kx + " + 2] = v_[2]; " + regs +
                     "[" + kx + " + 3] = v_[3];");
            em_.close();
            if (groups * 4 < count) {
              openSteps(count, groups * 4, count);
              em_.line(regs + "[" + kx + "] = " + operandValue(load, false) + ";");
              em_.close();
            }
          };
          const bool vectorA = !resident && count >= 4 && contiguousAlongSteps(loadA);
          const bool vectorB = count >= 4 && contiguousAlongSteps(loadB);
          if (vectorA) vectorLoads(loadA, "aq_");
          if (vectorB) vectorLoads(loadB, "bq_");
          if ((!resident && !vectorA) || !vectorB) {
            bool masked = openSteps(count);
            if (!resident && !vectorA) em_.line("aq_[" + kx + "] = " + operandValue(loadA, masked) + ";");
            if (!vectorB) em_.line("bq_[" + kx + "] = " + operandValue(loadB, masked) + ";");
            em_.close();
          }
          em_.line("#pragma unroll");
          em_.open("for (int " + kx + " = 0; " + kx + " < " + std::to_string(count) + "; ++" + kx + ")");
          em_.line(acc + " = __builtin_amdgcn_mfma_f32_16x16x4f32(" + (resident ? "am_" : "aq_") + "[" + kx + "], bq_[" + kx + "], " +
                   acc + ", 0, 0, 0);");
          em_.close();
        } else {
          bool masked = openSteps(count);
          em_.line("const float a_ = " + (resident ? std::string("am_[ks_]") : operandValue(loadA, masked)) + ";");
          em_.line("const float b_ = " + operandValue(loadB, masked) + ";");
          em_.line(acc + " = __builtin_amdgcn_mfma_f32_16x16x4f32(a_, b_, " + acc + ", 0, 0, 0);");
          em_.close();
        }
      };
      if (unevenSplit) {
        // the last slice is shorter: its own copy of the loop, chosen per wavefront
        em_.open("if (sl_ < " + std::to_string(split - 1) + ")");
        steps(stepsPerWave);
        em_.close();
        em_.open("else");
        steps(ksteps - (split - 1) * stepsPerWave);
        em_.close();
      } else {
        steps(stepsPerWave);
      }
      em_.close();
    };
    // Epilogue and store: a lane holds rows 4*lj_ .. 4*lj_+3 of column lm_.  Indices are clamped
    // to legal points, so the epilogue's loads need no guard: the four rows are finished first
    // (their loads issue together and, when they do not depend on the column, move out of the
    // tile loop), then stored under one test of the column.
    auto finish = [&](const std::string& acc, const std::string& columnOk = "nok_") {
      const bool mExact = groupExact(st_.mfmaM, MT, 16);
      em_.line(accType_.cName() + " out_[4];");
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int mpos_ = mt_ * 16 + 4 * lj_ + r_;");
      decodeGroup(st_.mfmaM, "mpos_", true, MT % 16 == 0);
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
      em_.open("if (" + columnOk + ")");
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("const int mpos_ = mt_ * 16 + 4 * lj_ + r_;");
      std::string mok = decodeGroup(st_.mfmaM, "mpos_", true, MT % 16 == 0);
      em_.line(storeStmt(mExact ? "true" : mok, "out_[r_]"));
      em_.close();
      em_.close();
    };
    // One quarter-tile pass, unit tl_ - fullTiles of the block: four surplus columns of one row tile.
    auto decodeQuarter = [&]() {
      const std::string Q = std::to_string(remPasses);
      em_.line("const int ru_ = tl_ - " + std::to_string(fullTiles) + ";");
      em_.line("const int rp_ = ru_ % " + Q + ", mt_ = (ru_ / " + Q + ") % " + std::to_string(numMT) + ", bt_ = ru_ / " +
               std::to_string(remPasses * numMT) + ";");
      em_.line("(void)rp_;");
      std::string bok = st_.mfmaBatch.empty() ? "true" : decodeGroup(st_.mfmaBatch, "bt_", true, true);
      em_.line("const bool bok_ = " + bok + ";");
      if (columnsCached) {
        cachedColumns();
        return;
      }
      em_.line("const int npos_ = " + std::to_string(numNTfull * 16) + " + 4 * rp_ + (threadIdx.x & 3);");
      em_.line("const bool nok_ = bok_ && " + decodeGroup(st_.mfmaN, "npos_", true, remCols % 4 == 0) + ";");
      em_.line("(void)nok_;");
    };
    auto quarterPass = [&]() {
      decodeQuarter();
      em_.line("__tc::floatx4 c_;");
      em_.open("");
      em_.line("const int mposa_ = mt_ * 16 + lm_;");
      em_.line("const bool moka_ = bok_ && " + decodeGroup(st_.mfmaM, "mposa_", true, MT % 16 == 0) + ";");
      em_.line("(void)moka_;");
      em_.line("float bq_[" + std::to_string(ksteps) + "];");
      if (!resident) em_.line("float aq_[" + std::to_string(ksteps) + "];");
      bool masked = openSteps(ksteps);
      if (!resident) em_.line("aq_[ks_] = " + operandValue(loadA, masked) + ";");
      em_.line("bq_[ks_] = " + operandValue(loadB, masked) + ";");
      em_.close();
      // four independent accumulators: a chain of dependent 4x4x1 instructions issues at a third of
      // the rate of independent ones
      em_.line("__tc::floatx4 cq_[4];");
      em_.line("#pragma unroll");
      em_.line("for (int q_ = 0; q_ < 4; ++q_) cq_[q_] = __tc::floatx4{0.0f, 0.0f, 0.0f, 0.0f};");
      em_.line("#pragma unroll");
      em_.open("for (int ks_ = 0; ks_ < " + std::to_string(ksteps) + "; ++ks_)");
      em_.line(std::string("cq_[ks_ & 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(") + (resident ? "am_" : "aq_") +
               "[ks_], bq_[ks_], cq_[ks_ & 3], 0, 0, 0);");
      em_.close();
      em_.line("c_ = (cq_[0] + cq_[1]) + (cq_[2] + cq_[3]);");
      // the four quarters of the reduction meet: lanes l, l ^ 16, l ^ 32, l ^ 48
      em_.line("#pragma unroll");
      em_.open("for (int r_ = 0; r_ < 4; ++r_)");
      em_.line("float v_ = c_[r_];");
      em_.line("v_ += __tc::laneXor32<16>(v_);");
      em_.line("v_ += __tc::laneXor32<32>(v_);");
      em_.line("c_[r_] = v_;");
      em_.close();
      em_.close();
      // rows of this lane in the quarter-tile layout; the first 16 lanes store
      em_.open("");
      em_.line("const int lj_ = " + quadOfLane + ";");
      em_.line("const bool nokq_ = nok_ && threadIdx.x < 16;");
      auto saved = hoistedLoads_;
      for (size_t h = 0; h < hoistedCount; ++h) hoistedLoads_[hoistedTexts[h]] = "er" + std::to_string(h) + "_[r_]";
      finish("c_", "nokq_");
      hoistedLoads_ = saved;
      em_.close();
    };
    // Which tile a wavefront works on, who multiplies and who finishes it.  Without a split
    // wavefront wv_ takes tiles wv_, wv_ + waves, ...; with one, wavefront wv_ takes slice
    // wv_ / tiles of the reduction of tile wv_ % tiles and slice 0 owns the tile.
    const std::string T = std::to_string(tiles), W = std::to_string(st_.waves), S = std::to_string(split);
    // Register blocking (reduction-tiled stages).  A wavefront that owns a rectangle of RM x RN
    // output tiles reads RM M-side and RN N-side operand values per reduction step for RM * RN
    // multiplications, and its accumulators take turns, so no multiplication waits for the one
    // before it (a chain of dependent 16x16x4 instructions issues every 43 cycles instead of
    // every 32 when a SIMD holds a single wavefront).  The wavefronts form a WM x WN grid over
    // the tiles of the block; without such a grid tiles are dealt round-robin and multiplied one
    // at a time.
    int64_t blockWM = 0, blockWN = 0;
    if (kTiled && split == 1 && BT == 1 && tiles % st_.waves == 0 && ceilDiv(tiles, st_.waves) <= 16) {
      int64_t bestCost = 0;
      for (int64_t wm = 1; wm <= st_.waves; ++wm) {
        if (st_.waves % wm != 0) continue;
        const int64_t wn = st_.waves / wm;
        if (numMT % wm != 0 || numNT % wn != 0) continue;
        const int64_t rm = numMT / wm, rn = numNT / wn;
        // operand registers of one reduction tile: (rm + rn) values per step
        if ((rm + rn) * stepsPerWave > 128) continue;
        if (blockWM == 0 || rm + rn < bestCost) {
          blockWM = wm;
          blockWN = wn;
          bestCost = rm + rn;
        }
      }
    }
    const bool registerBlocked = blockWM > 0;
    const int64_t RM = registerBlocked ? numMT / blockWM : 0, RN = registerBlocked ? numNT / blockWN : 0;
    const std::string tileDecl =
        split > 1 ? "const int tl_ = wv_ % " + T + ", sl_ = wv_ / " + T + ";"
        : registerBlocked
            ? "const int tl_ = ((wv_ / " + std::to_string(blockWN) + ") * " + std::to_string(RM) + " + j_ / " + std::to_string(RN) +
                  ") * " + std::to_string(numNT) + " + (wv_ % " + std::to_string(blockWN) + ") * " + std::to_string(RN) + " + j_ % " +
                  std::to_string(RN) + ";"
            : "const int tl_ = wv_ + j_ * " + W + ";";
    const std::string worksOnTile = split > 1 ? "sl_ < " + S : "tl_ < " + T;
    const std::string ownsTile = split > 1 ? "sl_ == 0" : "tl_ < " + T;
    const std::string partialAt = kSplitName() + "[((%s * " + T + " + tl_) * 64 + threadIdx.x) * 4]";
    auto partial = [&](const std::string& slice) {
      std::string t = partialAt;
      return t.replace(t.find("%s"), 2, slice);
    };
    // every wavefront of the block passes here: the partial tiles of slices 1.. go to LDS
    auto exchange = [&](const std::string& acc) {
      em_.line("if (sl_ > 0 && sl_ < " + S + ") *(__tc::floatx4*)&" + partial("(sl_ - 1)") + " = " + acc + ";");
      em_.line("__syncthreads();");
    };
    auto gather = [&](const std::string& acc) {
      em_.line("#pragma unroll");
      em_.open("for (int o_ = 0; o_ < " + std::to_string(split - 1) + "; ++o_)");
      em_.line(acc + " += *(const __tc::floatx4*)&" + partial("o_") + ";");
      em_.close();
    };
    // which wavefront takes the surplus tile rotates with the block, so that the blocks sharing a
    // compute unit load its four SIMDs evenly
    const std::string waveRotation =
        "const int wv_ = (threadIdx.y + blockIdx.x + blockIdx.y + blockIdx.z) % " + std::to_string(st_.waves) + ";";
    int opened = 0;
    em_.open("");
    ++opened;
    // Column indices ahead of the staging.  Decoding a column position into the indices of the
    // N-side variables divides by the tile extents (pixel -> row, column of a 14 x 14 image); for
    // an unrolled tile loop behind a staging copy that is done for all tiles of the wavefront
    // while the copy's loads are in flight, together with the N-side part of every element offset
    // (columnSumOf), and kept: an empty asm pins each value, the compiler would otherwise move the
    // arithmetic back behind the barrier, between the multiplications.  The code behind this point
    // is generated first, since it tells which sums it needs, and is appended to the pass.
    const int64_t unitsAll = quarterTiles ? fullTiles + remUnits : tiles;
    const bool cacheColumns = raisePriority && !kTiled && split == 1 && tilesPerWave <= 8 && !st_.mfmaN.empty();
    std::string headText;
    int headIndent = 0;
    if (cacheColumns) {
      em_.line(waveRotation);
      headText = em_.out.str();
      em_.out.str("");
      em_.out.clear();
      headIndent = em_.indent;
    }
    stagePromotions(false);
    columnsCached = cacheColumns;
    if (cacheColumns) {
      columnSums_ = true;
      columnVars_ = st_.mfmaN;
      columnCombos_.clear();
    }
    if (raisePriority) em_.line("__builtin_amdgcn_s_setprio(0);");
    auto emitColumnPass = [&]() {
      const std::string body = em_.out.str();
      const int tailIndent = em_.indent;
      em_.out.str("");
      em_.out.clear();
      em_.out << headText;
      em_.indent = headIndent;
      columnSums_ = false;
      columnsCached = false;
      // an index variable the body names outside its own declarations is handed over as well
      std::vector<bool> indexUsed;
      for (const auto& n : st_.mfmaN) {
        const std::string name = iv(var(n));
        size_t uses = 0, decls = 0;
        for (size_t at = body.find(name); at != std::string::npos; at = body.find(name, at + 1)) {
          const bool startsWord = at == 0 || !(std::isalnum(static_cast<unsigned char>(body[at - 1])) || body[at - 1] == '_');
          const size_t end = at + name.size();
          const bool endsWord = end >= body.size() || !(std::isalnum(static_cast<unsigned char>(body[end])) || body[end] == '_');
          if (!startsWord || !endsWord) continue;
          ++uses;
          // (its declaration from the cache and the cast that keeps an unused one quiet do not count)
          if (body.compare(end, 5, " = dn") == 0) ++decls;
          if (at >= 6 && body.compare(at - 6, 6, "(void)") == 0) ++decls;
        }
        indexUsed.push_back(uses > decls);
      }
      const std::string J = std::to_string(tilesPerWave);
      for (size_t i = 0; i < st_.mfmaN.size(); ++i) em_.line("int dn" + std::to_string(i) + "_[" + J + "];");
      for (size_t k = 0; k < columnCombos_.size(); ++k) em_.line("int ds" + std::to_string(k) + "_[" + J + "];");
      em_.line("bool dok_[" + J + "];");
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + J + "; ++j_)");
      em_.line("const int tl_ = wv_ + j_ * " + std::to_string(st_.waves) + ";");
      for (size_t i = 0; i < st_.mfmaN.size(); ++i) em_.line("dn" + std::to_string(i) + "_[j_] = 0;");
      for (size_t k = 0; k < columnCombos_.size(); ++k) em_.line("ds" + std::to_string(k) + "_[j_] = 0;");
      em_.line("dok_[j_] = false;");
      auto keep = [&]() {
        for (size_t i = 0; i < st_.mfmaN.size(); ++i) {
          if (indexUsed[i]) em_.line("dn" + std::to_string(i) + "_[j_] = " + iv(var(st_.mfmaN[i])) + ";");
        }
        for (size_t k = 0; k < columnCombos_.size(); ++k) {
          Affine a = columnCombos_[k];
          a.constant = 0;
          em_.line("ds" + std::to_string(k) + "_[j_] = " + affineStr(a) + ";");
        }
        em_.line("dok_[j_] = nok_;");
      };
      if (!quarterTiles || fullTiles > 0) {
        em_.open("if (tl_ < " + std::to_string(quarterTiles ? fullTiles : tiles) + ")");
        decodeTile();
        keep();
        em_.close();
      }
      if (quarterTiles) {
        em_.open(std::string(fullTiles > 0 ? "else " : "") + "if (tl_ < " + std::to_string(unitsAll) + ")");
        decodeQuarter();
        keep();
        em_.close();
      }
      for (size_t i = 0; i < st_.mfmaN.size(); ++i) {
        if (indexUsed[i]) em_.line("asm volatile(\"\" : \"+v\"(dn" + std::to_string(i) + "_[j_]));");
      }
      for (size_t k = 0; k < columnCombos_.size(); ++k) em_.line("asm volatile(\"\" : \"+v\"(ds" + std::to_string(k) + "_[j_]));");
      em_.close();
      em_.out << body;
      em_.indent = tailIndent;
      columnCombos_.clear();
      columnVars_.clear();
    };
    if (resident && residentFromLds) fillResident();
    if (!kTiled && split > 1) {
      em_.line(waveRotation);
      em_.line(tileDecl);
      em_.line("__tc::floatx4 c_ = {0.0f, 0.0f, 0.0f, 0.0f};");
      em_.open("if (" + worksOnTile + ")");
      decodeTile();
      if (!s.init) {
        em_.open("if (" + ownsTile + ")");
        loadExisting("c_");
        em_.close();
      }
      multiply("c_");
      em_.close();
      exchange("c_");
      em_.open("if (" + ownsTile + ")");
      ++opened;
      decodeTile();
      gather("c_");
      finish("c_");
    } else if (!kTiled) {
      if (!cacheColumns) em_.line(waveRotation);
      const int64_t units = unitsAll;
      if (tilesPerWave <= 8) {
        // few tiles per wavefront: unrolled, so that the operand reads of a tile can be scheduled
        // above the epilogue and the stores of the tile before it
        em_.line("#pragma unroll");
        em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
        ++opened;
        em_.line("const int tl_ = wv_ + j_ * " + std::to_string(st_.waves) + ";");
      } else {
        em_.open("for (int tl_ = wv_; tl_ < " + std::to_string(units) + "; tl_ += " + std::to_string(st_.waves) + ")");
        ++opened;
      }
      if (!quarterTiles || fullTiles > 0) {
        em_.open("if (tl_ < " + std::to_string(quarterTiles ? fullTiles : tiles) + ")");
        decodeTile();
        em_.line("__tc::floatx4 c_ = {0.0f, 0.0f, 0.0f, 0.0f};");
        if (!s.init) loadExisting("c_");
        multiply("c_");
        finish("c_");
        em_.close();
      }
      if (quarterTiles) {
        // (the quarter-tile passes continue the round-robin of the full tiles, so they go to the
        // wavefronts with the fewest full tiles)
        em_.open(std::string(fullTiles > 0 ? "else " : "") + "if (tl_ < " + std::to_string(units) + ")");
        quarterPass();
        em_.close();
      }
    } else {
      em_.line(waveRotation);
      em_.line("__tc::floatx4 cacc_[" + std::to_string(tilesPerWave) + "];");
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
      em_.line("cacc_[j_] = __tc::floatx4{0.0f, 0.0f, 0.0f, 0.0f};");
      if (!s.init) {
        em_.line(tileDecl);
        em_.open("if (" + ownsTile + ")");
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
      // (two copies of every array staged per reduction tile: the next tile is stored into the
      // other copy right after the multiplications, no barrier between reading and overwriting)
      bool twoCopies = pipelineK;
      for (const auto& p : st_.promotions) twoCopies &= !p.insideReductionTiles || p.buffers == 2;
      // Rotated pipeline (register-blocked stages with two LDS copies whose operands both come
      // from LDS).  With one or two wavefronts per SIMD that all pass the same barrier, nothing
      // multiplies while the block stores a tile, waits and reads its first operand values.  The
      // steps of a tile are therefore cut in two halves: the operand values of the first half of
      // tile t+1 are read right behind the barrier that publishes it, while the second half of
      // tile t (read before the barrier) is still being multiplied, and the stores of tile t+1
      // sit one step of multiplications ahead of that barrier.
      bool bothStaged = true;
      for (const ExprRef* l : {&loadA, &loadB}) {
        bool staged = false;
        for (const auto& p : st_.promotions) staged |= p.insideReductionTiles && p.tensor == (*l)->name;
        bothStaged &= staged;
      }
      const bool rotated = registerBlocked && pipelineK && twoCopies && bothStaged && stepsPerWave >= 2 && !forwardOf(loadA->name) &&
          !forwardOf(loadB->name);
      const int64_t halfSteps = stepsPerWave / 2;
      // Both operands float16: four consecutive steps of a lane (four values of its quarter of the
      // reduction tile per operand) are one v_mfma_f32_16x16x16_f16 - its lane group g supplies
      // k = 4g .. 4g+3, the group's four values, so the instruction adds exactly what four
      // 16x16x4 float steps add (products of halves are exact in float, the sums are float) at a
      // sixteenth of their issue time.  The operand registers then hold halves.
      const bool halfSteps16 = registerBlocked && st_.views.at(loadA->name).type.bits == 16 &&
          st_.views.at(loadB->name).type.bits == 16 && stepsPerWave % 4 == 0 && (!rotated || halfSteps % 4 == 0);
      const int64_t lead = halfSteps16 ? 4 : 1; // the multiplications kept between the stores and the barrier
      const std::string operandType = halfSteps16 ? "_Float16" : "float";
      // operand values of steps [first, last) of the wavefront's rectangle into ra_ / rb_
      auto readOperands = [&](int64_t first, int64_t last) {
        em_.open("");
        em_.line("const int bt_ = 0;");
        em_.line("(void)bt_;");
        std::string bok = st_.mfmaBatch.empty() ? "true" : decodeGroup(st_.mfmaBatch, "bt_", true, true);
        em_.line("const bool bok_ = " + bok + ";");
        em_.line("(void)bok_;");
        em_.line("#pragma unroll");
        em_.open("for (int a_ = 0; a_ < " + std::to_string(RM) + "; ++a_)");
        em_.line("const int mt_ = (wv_ / " + std::to_string(blockWN) + ") * " + std::to_string(RM) + " + a_;");
        em_.line("const int mposa_ = mt_ * 16 + lm_;");
        em_.line("const bool moka_ = bok_ && " + decodeGroup(st_.mfmaM, "mposa_", true, MT % 16 == 0) + ";");
        em_.line("(void)moka_;");
        {
          bool masked = openSteps(stepsPerWave, first, last);
          em_.line("ra_[a_][ks_] = " + operandValue(loadA, masked) + ";");
          em_.close();
        }
        em_.close();
        em_.line("#pragma unroll");
        em_.open("for (int b_ = 0; b_ < " + std::to_string(RN) + "; ++b_)");
        em_.line("const int nt_ = (wv_ % " + std::to_string(blockWN) + ") * " + std::to_string(RN) + " + b_;");
        em_.line("const int npos_ = nt_ * 16 + lm_;");
        em_.line("const bool nok_ = bok_ && " + decodeGroup(st_.mfmaN, "npos_", true, NT % 16 == 0) + ";");
        em_.line("(void)nok_;");
        {
          bool masked = openSteps(stepsPerWave, first, last);
          em_.line("rb_[b_][ks_] = " + operandValue(loadB, masked) + ";");
          em_.close();
        }
        em_.close();
        em_.close();
      };
      // the multiplications of steps [first, last), step by step over all tiles of the rectangle
      auto multiplySteps = [&](int64_t first, int64_t last) {
        if (first >= last) return;
        if (halfSteps16) {
          em_.line("#pragma unroll");
          em_.open("for (int ks_ = " + std::to_string(first) + "; ks_ < " + std::to_string(last) + "; ks_ += 4)");
          em_.line("#pragma unroll");
          em_.open("for (int a_ = 0; a_ < " + std::to_string(RM) + "; ++a_)");
          em_.line("const __tc::halfx4 av_ = {ra_[a_][ks_], ra_[a_][ks_ + 1], ra_[a_][ks_ + 2], ra_[a_][ks_ + 3]};");
          em_.line("#pragma unroll");
          em_.open("for (int b_ = 0; b_ < " + std::to_string(RN) + "; ++b_)");
          em_.line("const __tc::halfx4 bv_ = {rb_[b_][ks_], rb_[b_][ks_ + 1], rb_[b_][ks_ + 2], rb_[b_][ks_ + 3]};");
          em_.line("cacc_[a_ * " + std::to_string(RN) + " + b_] = __builtin_amdgcn_mfma_f32_16x16x16f16(av_, bv_, cacc_[a_ * " +
                   std::to_string(RN) + " + b_], 0, 0, 0);");
          em_.close();
          em_.close();
          em_.close();
          return;
        }
        em_.line("#pragma unroll");
        em_.open("for (int ks_ = " + std::to_string(first) + "; ks_ < " + std::to_string(last) + "; ++ks_)");
        em_.line("#pragma unroll");
        em_.open("for (int a_ = 0; a_ < " + std::to_string(RM) + "; ++a_)");
        em_.line("#pragma unroll");
        em_.open("for (int b_ = 0; b_ < " + std::to_string(RN) + "; ++b_)");
        em_.line("cacc_[a_ * " + std::to_string(RN) + " + b_] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra_[a_][ks_], rb_[b_][ks_], cacc_[a_ * " +
                 std::to_string(RN) + " + b_], 0, 0, 0);");
        em_.close();
        em_.close();
        em_.close();
      };
      if (rotated) {
        // Register stages of the staging copies: the loads of a tile are issued `stages` tiles
        // ahead of the stores that wait for them (a tile of 32 reduction values is multiplied
        // in about 0.4 us, a load that misses the L2 takes longer), one set of registers per
        // tile in flight; the tile loop is unrolled by that number so that every set and both
        // LDS copies are named statically.
        const int64_t numK = k0.numTiles;
        int64_t stages = 1;
        while (stages < 4 && 2 * stages * stagingRegs <= 64 && numK >= 4 * stages && numK % (2 * stages) == 0) stages *= 2;
        auto regs = [&](const Promotion& p, int64_t st) { return "pk" + std::to_string(st) + "_" + p.tensor + "_"; };
        em_.open("");
        ++opened;
        for (int64_t st = 0; st < stages; ++st) {
          for (const auto& p : st_.promotions) {
            if (p.insideReductionTiles) em_.line(copyRegisterDecl(p, regs(p, st)));
          }
        }
        em_.line(operandType + " ra_[" + std::to_string(RM) + "][" + std::to_string(stepsPerWave) + "];");
        em_.line(operandType + " rb_[" + std::to_string(RN) + "][" + std::to_string(stepsPerWave) + "];");
        auto loadTile = [&](const std::string& tile, int64_t st) {
          em_.open("");
          tileOverride[k0.name] = tile;
          for (const auto& p : st_.promotions) {
            if (!p.insideReductionTiles) continue;
            declareLows(p);
            emitCopyLoads(p, regs(p, st));
          }
          tileOverride.clear();
          em_.close();
        };
        auto storeTile = [&](const std::string& buffer, int64_t st) {
          writeBuffer_ = buffer;
          for (const auto& p : st_.promotions) {
            if (p.insideReductionTiles) emitCopyStores(p, regs(p, st));
          }
          writeBuffer_.clear();
        };
        auto readHalf = [&](const std::string& tile, const std::string& buffer, int64_t first, int64_t last) {
          em_.open("");
          tileOverride[k0.name] = tile;
          readBuffer_ = buffer;
          for (const auto& p : st_.promotions) {
            if (p.insideReductionTiles) declareLows(p);
          }
          readOperands(first, last);
          tileOverride.clear();
          readBuffer_.clear();
          em_.close();
        };
        // (the loads of the first tiles all leave before the first of them is waited for: one
        // memory latency ahead of the loop instead of two)
        for (int64_t j = 0; j < stages; ++j) loadTile(std::to_string(std::min(j, numK - 1)), j);
        em_.line("__syncthreads();");
        storeTile("0", 0);
        loadTile(std::to_string(std::min(stages, numK - 1)), 0);
        em_.line("__syncthreads();");
        for (const auto& p : st_.promotions) {
          if (p.insideReductionTiles) activePromotions_.insert(p.tensor);
        }
        readHalf("0", "0", 0, halfSteps);
        const std::string t0 = tk + "0_", NK = std::to_string(numK), ST = std::to_string(stages);
        em_.open("for (int " + t0 + " = 0; " + t0 + " < " + NK + "; " + t0 + " += " + ST + ")");
        for (int64_t d = 0; d < stages; ++d) {
          em_.open("");
          em_.line("const int " + tk + " = " + t0 + " + " + std::to_string(d) + ";");
          const bool staticCopy = stages % 2 == 0;
          const std::string cur = staticCopy ? std::to_string(d & 1) : "(" + tk + " & 1)";
          const std::string nxt = staticCopy ? std::to_string((d + 1) & 1) : "((" + tk + " + 1) & 1)";
          const int64_t nextStage = (d + 1) % stages;
          // second half of this tile's operand values, while the first half is multiplied
          readHalf(tk, cur, halfSteps, stepsPerWave);
          multiplySteps(0, halfSteps - lead);
          em_.line("__builtin_amdgcn_sched_barrier(0);");
          // (no branches in the loop body: with them the compiler waits for every load in flight
          // ahead of a store instead of the oldest ones.  Past the last tile the loads fetch the
          // last tile again and the stores and reads move values nobody multiplies.)
          storeTile(nxt, nextStage);
          loadTile("min(" + tk + " + " + std::to_string(1 + stages) + ", " + std::to_string(numK - 1) + ")", nextStage);
          em_.line("__builtin_amdgcn_sched_barrier(0);");
          // (one step of multiplications between the stores and the barrier that waits for them)
          multiplySteps(halfSteps - lead, halfSteps);
          // (and they stay there: the scheduler would lift the barrier, which is no memory
          // operation to the multiplications, above all but one of them)
          em_.line("__builtin_amdgcn_sched_barrier(0);");
          em_.line("__syncthreads();");
          readHalf("min(" + tk + " + 1, " + std::to_string(numK - 1) + ")", nxt, 0, halfSteps);
          em_.line("__builtin_amdgcn_sched_barrier(0);"); // (the reads stay ahead of the multiplications that cover them)
          multiplySteps(halfSteps, stepsPerWave);
          em_.close();
        }
        em_.close();
      } else {
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
          if (twoCopies) writeBuffer_ = "0";
          for (const auto& p : st_.promotions) {
            if (p.insideReductionTiles) emitCopyStores(p, "pk_" + p.tensor + "_");
          }
          writeBuffer_.clear();
          em_.close();
        }
        em_.open("for (int " + tk + " = 0; " + tk + " < " + std::to_string(k0.numTiles) + "; ++" + tk + ")");
        if (pipelineK && twoCopies) {
          readBuffer_ = "(" + tk + " & 1)";
          writeBuffer_ = "((" + tk + " + 1) & 1)";
        }
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
          // (the loads of the next tile are issued here, a whole tile of multiplications ahead of
          // the stores that wait for them: the instruction scheduler would otherwise sink them next
          // to those stores and every wavefront would sit out the memory latency once per tile)
          em_.line("__builtin_amdgcn_sched_barrier(0);");
          for (const auto& p : st_.promotions) {
            if (!p.insideReductionTiles) continue;
            declareLows(p);
            activePromotions_.insert(p.tensor);
          }
        } else {
          stagePromotions(true);
        }
        if (registerBlocked) {
          em_.line(operandType + " ra_[" + std::to_string(RM) + "][" + std::to_string(stepsPerWave) + "];");
          em_.line(operandType + " rb_[" + std::to_string(RN) + "][" + std::to_string(stepsPerWave) + "];");
          // the operand values of the whole reduction tile first, then the multiplications
          readOperands(0, stepsPerWave);
          multiplySteps(0, stepsPerWave);
        } else {
          em_.line("#pragma unroll");
          em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
          em_.line(tileDecl);
          em_.open("if (" + worksOnTile + ")");
          decodeTile();
          multiply("cacc_[j_]");
          em_.close();
          em_.close();
        }
        if (pipelineK) {
          if (!twoCopies) em_.line("__syncthreads();");
          else em_.line("__builtin_amdgcn_sched_barrier(0);"); // (nor may the stores rise among the multiplications)
          em_.open("if (more_)");
          for (const auto& p : st_.promotions) {
            if (p.insideReductionTiles) emitCopyStores(p, "pk_" + p.tensor + "_");
          }
          em_.close();
        }
        readBuffer_.clear();
        writeBuffer_.clear();
        em_.close();
      }
      if (split > 1) {
        em_.open("");
        em_.line(tileDecl);
        exchange("cacc_[0]");
        em_.close();
      }
      em_.line("#pragma unroll");
      em_.open("for (int j_ = 0; j_ < " + std::to_string(tilesPerWave) + "; ++j_)");
      ++opened;
      em_.line(tileDecl);
      em_.open("if (" + ownsTile + ")");
      ++opened;
      decodeTile();
      if (split > 1) gather("cacc_[j_]");
      finish("cacc_[j_]");
    }
    closeN(opened);
    // inside loops the partial tiles are written again: not before every owner has read them
    if (split > 1 && (kc_.kernelLoops || stageTileLoops_)) em_.line("__syncthreads();");
    if (cacheColumns) emitColumnPass();
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
      stageTileLoops_ = openedTiles > 1;
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
    // footprints of the block tile are staged ahead of per-thread loops that stay loops
    stageTileLoops_ = opened > 1;
    stagedAheadOfPointLoops_ = false;
    if (!st_.promotions.empty() && !fullRegisterTile()) {
      if (suppressCopy) {
        for (const auto& p : st_.promotions) declareLows(p);
      } else {
        stageFootprints(false);
        for (const auto& p : st_.promotions) activePromotions_.erase(p.tensor);
      }
      stagedAheadOfPointLoops_ = true;
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
  bool stageTileLoops_ = false; // the stage's code sits inside tile loops of its own
  bool kSplitAllowed_ = true;   // LDS has room for the partial tiles of a split reduction
  bool copiedBefore_ = false;   // this stage has already written LDS once
  bool stagedAheadOfPointLoops_ = false; // the footprints were staged before the per-thread loops opened
  const StageStmt* promotedPointwise_ = nullptr; // statement of a reduction-free stage that reads staged footprints
  std::string cacheSlot_;
  int clampId_ = 0;
};

