// Minimal synchronisation of a sequence of kernel stages.
//
// Role of the reference's findBestSyncConfigInSeq / insertBestSyncInSeq
// (tc/core/polyhedral/cuda/mapped_scop.cc:580-770): the children of a sequence run one after the
// other inside every block, optionally inside a sequential loop, and each pair of children needs a
// synchronisation of some level somewhere between them (none, the threads of one wavefront, the
// whole block).  The result is the cheapest set of barriers that satisfies every pair, cost
// compared as (number of block barriers, number of wavefront barriers).  A wavefront here has 64
// lanes (constructThreadToWarp uses 32, mapped_scop.cc:504-524).
//
// Unlike the reference, which splits ranges greedily around the strictest requirement when the
// sequence sits in a loop, the search below is exact for both the straight-line and the cyclic
// case: a barrier position on the cycle is fixed first, which opens the cycle into a line, and the
// line is solved by a dynamic programme over (last block barrier, last barrier of any level).
#pragma once
#include <algorithm>
#include <array>
#include <cstdint>
#include <utility>
#include <vector>

namespace tc {
namespace mapper {

enum class SyncLevel : int { None = 0, Wave = 1, Block = 2 };

// need[i][k]: level required between child i and child (i + k) % n.  k >= 1 with i + k < n is a
// pair of the same pass over the sequence; when the sequence is the body of a sequential loop
// (cyclic), k = 0 is child i against itself in the next iteration and i + k >= n is child i
// against child (i + k) - n of the next iteration.  Entries that do not apply are ignored.
using SyncNeeds = std::vector<std::vector<int>>;

// (position p, level): a barrier after child p; p = n - 1 is the end of the loop body.
using SyncList = std::vector<std::pair<int, SyncLevel>>;

namespace detail {

struct Interval {
  int first, last; // barrier positions (gaps) first..last must hold one barrier of >= level
  int level;
};

using Cost = std::pair<int, int>; // (block barriers, wavefront barriers)
constexpr int kInf = 1 << 20;

// Exact cover of intervals on a line of `m` gaps.  Returns false when an interval is empty.
inline bool solveLine(int m, const std::vector<Interval>& intervals, Cost& best, std::vector<int>& levels) {
  for (const auto& iv : intervals) {
    if (iv.first > iv.last) return false;
  }
  // state after deciding gaps 0..g-1: lb = last gap holding a block barrier + 1 (0: none),
  // la = last gap holding any barrier + 1
  const int S = m + 1;
  auto idx = [&](int lb, int la) { return lb * S + la; };
  std::vector<std::vector<Cost>> cost(m + 1, std::vector<Cost>(S * S, Cost{kInf, kInf}));
  std::vector<std::vector<std::array<int, 3>>> from(m + 1, std::vector<std::array<int, 3>>(S * S, {{-1, -1, -1}}));
  cost[0][idx(0, 0)] = {0, 0};
  // intervals grouped by their last gap, checked as soon as that gap is decided
  std::vector<std::vector<const Interval*>> endingAt(m);
  for (const auto& iv : intervals) endingAt[iv.last].push_back(&iv);
  for (int g = 0; g < m; ++g) {
    for (int lb = 0; lb <= g; ++lb) {
      for (int la = lb; la <= g; ++la) {
        Cost c = cost[g][idx(lb, la)];
        if (c.first >= kInf) continue;
        for (int lev = 0; lev <= 2; ++lev) {
          int nlb = lev == 2 ? g + 1 : lb;
          int nla = lev >= 1 ? g + 1 : la;
          bool ok = true;
          for (const Interval* iv : endingAt[g]) {
            int lastOk = iv->level == 2 ? nlb : nla;
            ok &= lastOk >= iv->first + 1;
          }
          if (!ok) continue;
          Cost nc{c.first + (lev == 2), c.second + (lev == 1)};
          Cost& slot = cost[g + 1][idx(nlb, nla)];
          if (nc < slot) {
            slot = nc;
            from[g + 1][idx(nlb, nla)] = {{lb, la, lev}};
          }
        }
      }
    }
  }
  best = {kInf, kInf};
  int bestState = -1;
  for (int s = 0; s < S * S; ++s) {
    if (cost[m][s] < best) {
      best = cost[m][s];
      bestState = s;
    }
  }
  if (bestState < 0) return false;
  levels.assign(m, 0);
  int lb = bestState / S, la = bestState % S;
  for (int g = m; g > 0; --g) {
    auto f = from[g][idx(lb, la)];
    levels[g - 1] = f[2];
    lb = f[0];
    la = f[1];
  }
  return true;
}

} // namespace detail

inline SyncList findBestSyncs(const SyncNeeds& need, bool cyclic) {
  using namespace detail;
  const int n = static_cast<int>(need.size());
  SyncList out;
  if (n == 0) return out;
  auto levelOf = [&](int i, int k) { return k < static_cast<int>(need[i].size()) ? need[i][k] : 0; };
  if (!cyclic) {
    std::vector<Interval> intervals;
    for (int i = 0; i < n; ++i) {
      for (int k = 1; i + k < n; ++k) {
        if (levelOf(i, k) > 0) intervals.push_back({i, i + k - 1, levelOf(i, k)});
      }
    }
    Cost c;
    std::vector<int> levels;
    if (n > 1 && solveLine(n - 1, intervals, c, levels)) {
      for (int g = 0; g < n - 1; ++g) {
        if (levels[g]) out.emplace_back(g, static_cast<SyncLevel>(levels[g]));
      }
    }
    return out;
  }
  // Cyclic: gaps 0..n-1 on a circle, gap n-1 closes the loop body.  Requirement (i, k) covers the
  // gaps i, i+1, ..., i+k-1 (mod n); k = 0 covers the whole circle.
  struct Arc {
    int start, len, level;
  };
  std::vector<Arc> arcs;
  int maxLevel = 0;
  for (int i = 0; i < n; ++i) {
    for (int k = 0; k < n; ++k) {
      int lev = levelOf(i, k);
      if (lev <= 0) continue;
      arcs.push_back({i, k == 0 ? n : k, lev});
      maxLevel = std::max(maxLevel, lev);
    }
  }
  if (arcs.empty()) return out;
  // Some barrier of the strictest level must exist: fix its gap `cut`; arcs through the cut are
  // satisfied, the others lie on the line of gaps cut+1, ..., cut+n-1.
  Cost best{kInf, kInf};
  std::vector<int> bestLevels;
  int bestCut = -1;
  for (int cut = 0; cut < n; ++cut) {
    std::vector<Interval> intervals;
    for (const auto& a : arcs) {
      int rel = ((a.start - (cut + 1)) % n + n) % n; // position of the arc's first gap on the line
      if (rel + a.len - 1 >= n - 1) continue;        // reaches the cut (line position n-1)
      intervals.push_back({rel, rel + a.len - 1, a.level});
    }
    Cost c;
    std::vector<int> levels;
    if (!solveLine(n - 1, intervals, c, levels)) continue;
    c.first += maxLevel == 2;
    c.second += maxLevel == 1;
    if (c < best) {
      best = c;
      bestLevels = levels;
      bestCut = cut;
    }
  }
  if (bestCut < 0) return out;
  std::vector<int> onCircle(n, 0);
  onCircle[bestCut] = maxLevel;
  for (int g = 0; g < n - 1; ++g) onCircle[(bestCut + 1 + g) % n] = bestLevels[g];
  for (int g = 0; g < n; ++g) {
    if (onCircle[g]) out.emplace_back(g, static_cast<SyncLevel>(onCircle[g]));
  }
  return out;
}

// true when `syncs` satisfies every requirement (used by tests and debug checks)
inline bool syncsAreSufficient(const SyncNeeds& need, bool cyclic, const SyncList& syncs) {
  const int n = static_cast<int>(need.size());
  std::vector<int> at(std::max(n, 1), 0);
  for (const auto& s : syncs) at[s.first] = std::max(at[s.first], static_cast<int>(s.second));
  for (int i = 0; i < n; ++i) {
    for (int k = 0; k < static_cast<int>(need[i].size()) && k < n; ++k) {
      int lev = need[i][k];
      if (lev <= 0) continue;
      if (!cyclic && (k == 0 || i + k >= n)) continue;
      int len = k == 0 ? n : k;
      bool ok = false;
      for (int g = 0; g < len; ++g) ok |= at[(i + g) % n] >= lev;
      if (!ok) return false;
    }
  }
  return true;
}

} // namespace mapper
} // namespace tc
