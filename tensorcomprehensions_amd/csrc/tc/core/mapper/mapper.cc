#include "tc/core/mapper/mapper.h"
#include "tc/core/mapper/sync_placement.h"

#include <limits>
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
  return t.bits == 64 ? s : t.bits == 16 ? "((_Float16)" + s + "f)" : s + "f";
}

int64_t ceilDiv(int64_t a, int64_t b) {
  return (a + b - 1) / b;
}

const char* axisName(int a) {
  return a == 0 ? "x" : a == 1 ? "y" : "z";
}

#include "tc/core/mapper/stage_builder.h"
#include "tc/core/mapper/stage_codegen.h"

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
      TC_CHECK_GT(v.extent, 0) << "loop variable " << v.name << " has no points";
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
  // One copy per kernel: a later stage whose footprint of a tensor is the one an earlier stage has
  // staged (same box, same origin, fixed for the whole kernel-level iteration) reads the earlier
  // stage's array.  Staged tensors are inputs of the TC, so nothing in the kernel changes them.
  {
    std::map<std::string, std::string> staged; // footprint key -> LDS array of the first stage that stages it
    for (size_t i = 0; i < gens.size(); ++i) {
      for (auto& p : gens[i].mutablePromotions()) {
        if (!gens[i].footprintFixedPerKernelIteration(p)) continue;
        std::string key = gens[i].footprintKey(p);
        auto found = staged.find(key);
        if (found == staged.end()) {
          staged.emplace(key, p.ldsName);
        } else {
          p.sharedWithEarlierStage = true;
          p.ldsName = found->second;
          ldsBudget += p.elems * k.stages[i].views.at(p.tensor).type.bytes();
        }
      }
    }
  }
  // Producer -> consumer through a register (usePrivateMemory): a block-wide reduction along
  // threadIdx.x leaves its result in every thread of the row.  When the element a thread has just
  // finished is the very element every later read of that tensor in the kernel asks of it, the
  // readers use the register (the reference promotes such written scalars to registers,
  // memory_promotion_heuristic.cc:581-616).  That holds when each subscript, on both sides, is one
  // parallel variable that the two stages tile alike at kernel level and spread alike over the
  // blocks and over threadIdx.y/z with one point per thread.
  std::vector<std::string> forwardDecls;
  if (kc.opts.usePrivateMemoryValue) {
    auto findVar = [](const StagePlan& st, const std::string& name, int* pos) -> const LoopVar* {
      for (size_t v = 0; v < st.vars.size(); ++v) {
        if (st.vars[v].name == name) {
          *pos = static_cast<int>(v);
          return &st.vars[v];
        }
      }
      return nullptr;
    };
    // the single variable of a subscript `v + c`; null otherwise
    auto plainVar = [&](const StagePlan& st, const ExprRef& e, int* pos, int64_t* constant) -> const LoopVar* {
      Affine a = ir::toAffine(e);
      if (!a.valid) return nullptr;
      const LoopVar* found = nullptr;
      for (const auto& c : a.coef) {
        if (c.second == 0) continue;
        if (c.second != 1 || found) return nullptr;
        found = findVar(st, c.first, pos);
        if (!found) return nullptr;
      }
      *constant = a.constant;
      return found;
    };
    for (size_t i = 0; i + 1 < gens.size(); ++i) {
      const StagePlan& prod = k.stages[i];
      const std::string& t = prod.tensor;
      if (!prod.threadReduction || prod.atomic || prod.mfma || prod.accCount != 1) continue;
      // the first stage that writes the tensor; later ones may update the value in place (below)
      bool first = true;
      for (size_t j = 0; j < i; ++j) first &= k.stages[j].tensor != t;
      // (an epilogue of the producer may re-read the element it is finishing: its running value)
      bool readsOtherElements = false;
      for (const auto& stmt : prod.stmts) {
        visit(stmt.rhs, [&](const ExprRef& e) {
          if (e->kind != Expr::Load || e->name != t) return;
          bool same = e->args.size() == prod.lhsSubs.size();
          for (size_t d = 0; same && d < e->args.size(); ++d) same = sameExpr(e->args[d], prod.lhsSubs[d]);
          readsOtherElements |= !same;
        });
      }
      if (!first || readsOtherElements) continue;
      // the producer's side: one point per thread, rows along threadIdx.y/z only
      std::vector<const LoopVar*> pvars;
      std::vector<int> ppos;
      std::vector<int64_t> pconst;
      bool ok = true;
      bool axisUsed[3] = {false, false, false};
      for (const auto& sub : prod.lhsSubs) {
        int pos = -1;
        int64_t c = 0;
        const LoopVar* v = plainVar(prod, sub, &pos, &c);
        ok = ok && v && !v->reduction && !v->vectorLane && v->perThread == 1 && v->threadAxis != 0 &&
            (pos < k.sharedDepth || v->numTiles == 1);
        if (!ok) break;
        if (v->threadAxis > 0) axisUsed[v->threadAxis] = true;
        pvars.push_back(v);
        ppos.push_back(pos);
        pconst.push_back(c);
      }
      // a row of threads that works on no element of the tensor reduces nothing but identities
      for (int a = 1; a < 3 && ok; ++a) ok = k.block[a] == 1 || axisUsed[a];
      // A later stage addresses the element this thread holds: the same variable of the same
      // tiling in every subscript.  Where the producer's variable is on no thread axis, every
      // thread holds the value of the block's one point along it, and the reader's variable may
      // sit on a thread axis: its threads beyond the point compute on the clamped index.
      auto sameElement = [&](const StagePlan& cons, const std::vector<ExprRef>& subs) {
        bool same = subs.size() == pvars.size();
        for (size_t d = 0; same && d < pvars.size(); ++d) {
          int pos = -1;
          int64_t c = 0;
          const LoopVar* v = plainVar(cons, subs[d], &pos, &c);
          const LoopVar* w = pvars[d];
          same = v && c == pconst[d] && !v->reduction && !v->vectorLane && v->perThread == 1 && v->min == w->min &&
              v->extent == w->extent && v->tile == w->tile && v->numTiles == w->numTiles &&
              v->blockAxis == w->blockAxis && v->gridExtent == w->gridExtent &&
              (v->threadAxis == w->threadAxis || (w->threadAxis < 0 && v->tile == 1)) &&
              (v->numTiles == 1 || (pos == ppos[d] && pos < k.sharedDepth));
        }
        return same;
      };
      bool anyReader = false;
      int lastWriter = static_cast<int>(i);
      for (size_t j = i + 1; j < gens.size() && ok; ++j) {
        const StagePlan& cons = k.stages[j];
        const bool writes = cons.tensor == t;
        if (!writes && !tensorsRead(cons).count(t)) continue;
        anyReader = true;
        ok = cons.views.at(t).extents == prod.views.at(t).extents;
        if (writes) {
          // an update in place of the value the threads hold: pointwise, one element per thread
          bool pointwise = !cons.atomic && !cons.mfma && !cons.threadReduction && cons.accCount == 1;
          for (const auto& stmt : cons.stmts) pointwise &= stmt.redVars.empty();
          ok = ok && pointwise && sameElement(cons, cons.lhsSubs);
          lastWriter = static_cast<int>(j);
        }
        for (const auto& stmt : cons.stmts) {
          visit(stmt.rhs, [&](const ExprRef& e) {
            if (!ok || e->kind != Expr::Load || e->name != t) return;
            ok = sameElement(cons, e->args);
          });
        }
      }
      if (!anyReader || !ok) continue;
      KernelCtx::RegisterForward f;
      f.producer = static_cast<int>(i);
      f.lastWriter = lastWriter;
      f.name = "rfwd" + std::to_string(i) + "_" + t;
      forwardDecls.push_back(prod.views.at(t).type.cName() + " " + f.name + ";");
      kc.registerForwards[t] = f;
    }
  }
  // Producer -> consumer through LDS (useSharedMemory): a tensor exactly one stage of the kernel
  // writes and later stages read, when every reader's box of one kernel-level iteration lies inside
  // the producer's and that box fits what is left of LDS.  Stages see the tensor through views that
  // may merge dimensions differently: only identical views are matched.
  if (kc.opts.useSharedMemoryValue) {
    for (size_t i = 0; i + 1 < gens.size(); ++i) {
      const StagePlan& prod = k.stages[i];
      const std::string& t = prod.tensor;
      bool sole = true;
      for (size_t j = 0; j < k.stages.size(); ++j) sole &= j == i || k.stages[j].tensor != t;
      if (!sole || tensorsRead(prod).count(t) || kc.registerForwards.count(t)) continue;
      auto wbox = gens[i].writeBox();
      if (!wbox.valid) continue;
      bool anyReader = false, ok = true;
      for (size_t j = i + 1; j < gens.size() && ok; ++j) {
        if (!tensorsRead(k.stages[j]).count(t)) continue;
        anyReader = true;
        ok = k.stages[j].views.at(t).extents == prod.views.at(t).extents;
        auto rbox = ok ? gens[j].readBox(t) : StageCodegen::IterationBox();
        ok = ok && rbox.valid && rbox.low.size() == wbox.low.size();
        for (size_t d = 0; ok && d < wbox.low.size(); ++d) {
          int64_t delta = rbox.low[d].constant - wbox.low[d].constant;
          ok = rbox.low[d].coef == wbox.low[d].coef && delta >= 0 && delta + rbox.extents[d] <= wbox.extents[d];
        }
      }
      if (!anyReader || !ok) continue;
      KernelCtx::Forward f;
      f.producer = static_cast<int>(i);
      f.ldsName = "fwd" + std::to_string(i) + "_" + t;
      f.extents = wbox.extents;
      // pitches: one that is a multiple of the 32 banks puts the lanes (or the four lane groups
      // of a matrix-core operand read) that step along its dimension onto the same banks; four
      // elements more spread them and keep rows 16-byte aligned
      f.strides.assign(wbox.extents.size(), 1);
      for (size_t d = wbox.extents.size(); d-- > 1;) {
        f.strides[d - 1] = f.strides[d] * wbox.extents[d];
        if (f.strides[d - 1] % 32 == 0 && wbox.extents[d - 1] > 1) f.strides[d - 1] += 4;
      }
      f.elems = wbox.extents.empty() ? 1 : f.strides[0] * wbox.extents[0];
      int64_t bytes = f.elems * prod.views.at(t).type.bytes();
      if (bytes > ldsBudget) continue;
      ldsBudget -= bytes;
      for (const auto& low : wbox.low) f.lows.push_back(StageCodegen::tileAffineStr(low));
      kc.forwards[t] = f;
    }
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
          if (e->kind != Expr::Load || kc.registerForwards.count(e->name)) return; // (already in a register)
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
              if (m->kind != Expr::Load || !found.empty() || kc.registerForwards.count(m->name)) return;
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
  {
    // buffer descriptors (base, size in bytes, raw 32-bit data format) of the results that are
    // stored with write-through
    std::set<std::string> through;
    for (size_t i = 0; i < gens.size(); ++i) {
      if (gens[i].streamedStore()) through.insert(k.stages[i].tensor);
    }
    for (const auto& t : through) {
      em.line("const __amdgpu_buffer_rsrc_t " + StageCodegen::bufferName(t) + " = __builtin_amdgcn_make_buffer_rsrc((void*)p" +
              t + ", 0, " + std::to_string(gens[0].viewBytes(t)) + ", 0x00020000);");
    }
  }
  if (scratchElems > 0) {
    // one scratch area typed per use; sized for the widest element
    em.line("__shared__ double red_scratch_raw_[" + std::to_string(scratchElems) + "];");
  }
  for (auto& g : gens) g.emitLdsDecls();
  for (const auto& fw : kc.forwards) {
    em.line("__shared__ __attribute__((aligned(16))) " + k.stages[fw.second.producer].views.at(fw.first).type.cName() + " " +
            fw.second.ldsName + "[" + std::to_string(fw.second.elems) + "];");
  }
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
  kc.kernelLoops = !loops.empty();
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
  for (const auto& d : forwardDecls) em.line(d);
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
        // (a result the later stage takes from a register is no dependence through memory)
        // (of its writers the last one alone stores it)
        auto inRegister = [&](const std::string& t) { return kc.registerForwards.count(t) > 0; };
        bool conflict = (a.tensor == b.tensor && !inRegister(a.tensor)) ||
            (tensorsRead(a).count(b.tensor) && !inRegister(b.tensor)) ||
            (tensorsRead(b).count(a.tensor) && !inRegister(a.tensor));
        if (conflict && !gens[j].readsPrivatelyFrom(a)) need[i][j - i] = level;
      }
    }
    for (const auto& sy : findBestSyncs(need, opened > 0)) syncAfter[sy.first] = static_cast<int>(sy.second);
    // a producer's copy in LDS is overwritten by the next kernel-level iteration: not before the
    // readers of this one are done
    if (opened > 0 && !kc.forwards.empty()) syncAfter.back() = std::max(syncAfter.back(), level);
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

namespace {
// e + c with the constant folded into an existing "+ constant"
ExprRef addConstant(const ExprRef& e, int64_t c) {
  if (e->kind == Expr::IntImm) return mkInt(e->ival + c);
  if (e->kind == Expr::Binary && e->name == "+" && e->args[1]->kind == Expr::IntImm) {
    return addConstant(e->args[0], e->args[1]->ival + c);
  }
  return c == 0 ? e : mkBin("+", e, mkInt(c));
}

// The storage of an output starts at its inferred lower bound: element k of dimension d holds
// the point mins[d] + k, the way a Halide buffer with a non-zero min is addressed (the bounds
// are set in tc/core/tc2halide.cc:903).  Rewrites the function to zero-based outputs: an index
// variable that subscripts a shifted dimension on the left-hand side is shifted by the bound
// (range and every use), and every other subscript of such a tensor has the bound subtracted.
ir::Function withZeroBasedOutputs(const ir::Function& in) {
  ir::Function f = in;
  std::map<std::string, std::vector<int64_t>> mins;
  for (auto& t : f.outputs) {
    mins[t.name] = t.mins;
    std::fill(t.mins.begin(), t.mins.end(), 0);
  }
  for (auto& s : f.statements) {
    std::map<std::string, int64_t> shift;
    const auto& m = mins.at(s.tensor);
    for (size_t d = 0; d < s.lhsVars.size(); ++d) {
      auto it = shift.find(s.lhsVars[d]);
      TC_CHECK(it == shift.end() || it->second == m[d])
          << "index " << s.lhsVars[d] << " subscripts two dimensions of " << s.tensor << " with different lower bounds";
      shift[s.lhsVars[d]] = m[d];
    }
    for (const auto& sh : shift) {
      ir::Range& r = s.ranges.at(sh.first);
      r.min -= sh.second;
      r.max -= sh.second;
    }
    s.rhs = rewrite(s.rhs, [&](const ExprRef& e) -> ExprRef {
      if (e->kind == Expr::Var) {
        auto it = shift.find(e->name);
        return it == shift.end() || it->second == 0 ? nullptr : mkBin("+", e, mkInt(it->second));
      }
      if (e->kind == Expr::Load) {
        auto it = mins.find(e->name);
        if (it == mins.end()) return nullptr;
        auto c = std::make_shared<Expr>(*e);
        for (size_t d = 0; d < c->args.size(); ++d) c->args[d] = addConstant(c->args[d], -it->second[d]);
        return c;
      }
      return nullptr;
    });
  }
  return f;
}
// reductionBlocks: a reduction `O(p...) op=(!) rhs` is divided among blocks along its outermost
// reduction index r (extent E, `split` = the largest divisor of E not above `blocks`):
//     O(p...) = identity of op                       only for "op=!", a kernel of its own
//     O(p...) op= rhs[r := r + (E / split) * slice]   slice in 0:split, r in 0:E/split
// where `slice` becomes the outermost parallel variable of the second statement and its partial
// results are combined into O atomically.  Floating-point sums then depend on the order in which the
// blocks arrive (within the rounding of any other summation order); integer sums do not.
// The identity of a reduction operator as an expression of the given 32- or 64-bit type (values
// an integer literal cannot spell are formed by an operation: 0 - 1 for the largest uint64).
ExprRef identityExpr(ReduceOp op, const ScalarType& t) {
  auto imm = [&](double f, int64_t i) {
    auto e = std::make_shared<Expr>();
    e->kind = t.isFloat() ? Expr::FloatImm : Expr::IntImm;
    e->type = t;
    e->fval = f;
    e->ival = i;
    return ExprRef(e);
  };
  auto minus = [&](const ExprRef& a, const ExprRef& b) { return mkExpr(Expr::Binary, t, "-", {a, b}); };
  if (op == ReduceOp::Plus) return imm(0.0, 0);
  if (op == ReduceOp::Times) return imm(1.0, 1);
  const bool largest = op == ReduceOp::Min; // a minimum starts from the largest value of the type
  if (t.isFloat()) {
    double m = t.bits == 64 ? std::numeric_limits<double>::max() : static_cast<double>(std::numeric_limits<float>::max());
    return imm(largest ? m : -m, 0);
  }
  if (t.code == ScalarType::UInt) {
    if (!largest) return imm(0.0, 0);
    return t.bits == 64 ? minus(imm(0.0, 0), imm(0.0, 1)) : imm(0.0, (int64_t(1) << t.bits) - 1);
  }
  const int64_t top = t.bits == 64 ? std::numeric_limits<int64_t>::max() : (int64_t(1) << (t.bits - 1)) - 1;
  return largest ? imm(0.0, top) : minus(imm(0.0, -top), imm(0.0, 1));
}

ir::Function withSplitReductions(const ir::Function& in, int64_t blocks) {
  ir::Function f = in;
  f.statements.clear();
  int counter = 0;
  for (const auto& s : in.statements) {
    const ir::Tensor* t = in.find(s.tensor);
    bool ok = t && s.op != ReduceOp::None && !s.redVars.empty() && accessesTo(s, s.tensor).empty() &&
        (t->type.bits == 32 || t->type.bits == 64);
    int64_t split = 1, extent = 0;
    if (ok) {
      extent = s.ranges.at(s.redVars[0]).extent();
      for (int64_t d = std::min<int64_t>(blocks, extent); d >= 2; --d) {
        if (extent % d == 0) {
          split = d;
          break;
        }
      }
    }
    if (split < 2) {
      f.statements.push_back(s);
      continue;
    }
    std::string slice;
    do {
      slice = "slice" + std::to_string(counter++);
    } while (s.ranges.count(slice));
    if (s.init) {
      ir::Statement zero;
      zero.tensor = s.tensor;
      zero.lhsVars = s.lhsVars;
      zero.zeroing = true;
      for (const auto& v : s.lhsVars) zero.ranges[v] = s.ranges.at(v);
      zero.type = t->type;
      zero.tree = s.tree;
      zero.rhs = identityExpr(s.op, t->type);
      f.statements.push_back(zero);
    }
    ir::Statement part = s;
    part.init = false;
    part.atomic = true;
    part.sliceVar = slice;
    part.lhsVars.insert(part.lhsVars.begin(), part.sliceVar);
    part.ranges[part.sliceVar] = ir::Range{0, split - 1};
    const std::string r = s.redVars[0];
    const int64_t chunk = extent / split;
    ir::Range& rr = part.ranges.at(r);
    rr.max = rr.min + chunk - 1;
    part.rhs = rewrite(s.rhs, [&](const ExprRef& e) -> ExprRef {
      if (e->kind != Expr::Var || e->name != r) return nullptr;
      return mkBin("+", e, mkBin("*", mkVar(part.sliceVar), mkInt(chunk)));
    });
    f.statements.push_back(part);
  }
  return f;
}
} // namespace

namespace {
HipMappingOptions fillMappingOptions(const HipMappingOptions& given) {
  HipMappingOptions o = given;
  o.tile(std::vector<uint64_t>{1024}).unroll(4).matchLibraryCalls(false);
  o.mapToThreads(256).mapToBlocks(1 << 20).useSharedMemory(false).usePrivateMemory(false);
  o.vectorWidth(4).collapseContiguous(true).useMfma(false).prefetchShared(false);
  return o;
}
} // namespace

MappedProgram mapToHip(
    const ir::Function& given,
    const HipMappingOptions& optionsIn,
    const std::string& specializedName,
    const DeviceLimits& limits) {
  // Range inference accepts `where i in 8:4` and reports a negative extent, as the reference's does
  // (test/test_inference.cc:498-511: "silently infers a negative size"); nothing can be launched
  // over such a range.
  for (const auto& s : given.statements) {
    for (const auto& r : s.ranges) {
      if (r.second.max < r.second.min) {
        throw lang::errorAt(s.tree) << "Empty range for variable " << r.first << ": " << r.second.min << ":" << r.second.max + 1;
      }
    }
  }
  bool shifted = false;
  for (const auto& t : given.outputs) {
    for (auto m : t.mins) shifted |= m != 0;
  }
  const ir::Function zeroBased = shifted ? withZeroBasedOutputs(given) : ir::Function();
  const bool divided = optionsIn.reductionBlocksValue > 1;
  const ir::Function dividedSums =
      divided ? withSplitReductions(shifted ? zeroBased : given, optionsIn.reductionBlocksValue) : ir::Function();
  const ir::Function& f = divided ? dividedSums : shifted ? zeroBased : given;
  // 1. stages
  std::vector<RawStage> raw;
  bool allowStageFusion = optionsIn.generic.intraTileScheduleOptions.fusionStrategy != FusionStrategy::Min ||
      optionsIn.generic.outerScheduleOptions.fusionStrategy != FusionStrategy::Min;
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
  FusionStrategy fs = optionsIn.generic.outerScheduleOptions.fusionStrategy;
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
  // Loop variables and size parameters are 32-bit: every single extent must fit; a tensor as a
  // whole may hold 2^31 elements or more, element offsets are then formed in 64 bits.
  int64_t maxNumel = 0;
  for (const auto* ts : {&f.inputs, &f.outputs}) {
    for (const auto& t : *ts) {
      maxNumel = std::max(maxNumel, t.numel());
      for (auto e : t.extents) {
        TC_CHECK_LT(e, (1LL << 31)) << "tensor " << t.name << " has a dimension of 2^31 or more elements; not supported";
      }
    }
  }
  const bool wide = maxNumel >= (1LL << 31);

  // The fill that precedes a divided sum: all dimensions merged, four elements per thread, 256
  // threads, as many blocks as that takes.
  HipMappingOptions fillOptions = fillMappingOptions(optionsIn);
  std::vector<const HipMappingOptions*> kernelOptions;
  bool anyThreadReduction = false;
  std::vector<std::unique_ptr<Emitter>> bodies;
  for (size_t gi = 0; gi < groups.size(); ++gi) {
    const bool fill = groups[gi].stages.size() == 1 && raw[groups[gi].stages[0]].first().zeroing;
    const HipMappingOptions& options = fill ? fillOptions : optionsIn;
    kernelOptions.push_back(&options);
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
  for (size_t ki = 0; ki < prog.kernels.size(); ++ki) {
    KernelPlan& k = prog.kernels[ki];
    KernelCtx kc{f, *kernelOptions[ki], k};
    kc.wide = wide;
    if (wide) kc.idx = "int64";
    mapKernel(kc, limits);
    for (const auto& st : k.stages) anyThreadReduction |= st.threadReduction || st.atomic;
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
