// Autotuner: searches mapping options by compiling and timing candidates on the device.
//
// Structure of the reference's harness (tc/autotuner/autotuner.h:37-161, autotuner-inl.h:37-518):
// per generation, a pool of compile threads walks the population with an atomic cursor and
// queues (executor | nullptr, candidate); one evaluation thread per device pops the queue,
// prunes hopeless candidates, profiles the rest ten times and records the median in the
// OptionsCache and on the candidate; the search strategy then breeds the next generation.
// SIGINT finishes the current generation and returns the best so far; SIGTERM aborts.
#pragma once
#include <limits>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cmath>
#include <csignal>
#include <map>
#include <deque>
#include <iostream>
#include <mutex>
#include <set>
#include <thread>
#include <unordered_map>

#include "tc/autotuner/genetic_search.h"
#include "tc/autotuner/options_cache.h"
#include "tc/autotuner/utils.h"
#include "tc/core/compiler.h"
#include "tc/core/hip/hip.h"
#include "tc/core/hip/hip_backend.h"
#include "tc/core/flags.h"
#include "tc/lang/parser.h"
#include "tc/lang/sema.h"

namespace tc {
namespace autotune {

struct TunerSettings {
  size_t generations = flags().tuner_gen_generations;
  size_t populationSize = flags().tuner_gen_pop_size;
  uint8_t crossOverRate = static_cast<uint8_t>(flags().tuner_gen_crossover_rate);
  uint8_t mutationRate = static_cast<uint8_t>(flags().tuner_gen_mutation_rate);
  size_t numberElites = flags().tuner_gen_number_elites;
  size_t threads = flags().tuner_threads;
  uint64_t minLaunchTotalThreads = flags().tuner_min_launch_total_threads;
  size_t maxUnroll = 256;
  int64_t seed = -1;
  bool verbose = flags().debug_tuner;
  size_t restoreNumber = flags().tuner_gen_restore_number;
  std::string cacheFile; // when set: seeds the first generation from it and appends the result
  // candidates doing more than this many times the per-thread work of the best one are not run
  double maxSerialDepthRatio = 256.0;
  // generation 0 also holds a few structured variants of the first base mapping (streaming,
  // row-reduction and matrix-core shapes); the search then starts from more than one basin
  bool seedHeuristics = true;
  // Half of the random members of generation 0 are drawn from what the output shape suggests
  // (structuredRandomMembers) instead of uniformly from the value sets; 0 = the reference's
  // uniform draw for all of them.
  bool structuredRandom = true;
  // after the last generation: rounds of one-gene steps around the best candidate (every gene
  // moved to its neighbouring values, one at a time); a round that finds nothing better ends it
  size_t refinementRounds = 2;
  // Options the mapper of this backend gives no meaning to (fixParametersBeforeScheduling,
  // tileImperfectlyNested, privateDepth: they exist for the reference's isl scheduler and its
  // promotion heuristic) keep the value of the first base mapping instead of being searched.
  bool fixInertParameters = true;
  // A bred candidate that the mapper refuses, or that maps to kernels this run has already
  // measured (an unmutated survivor, a child of near-identical parents, a mutation of an option
  // that does not apply), is mutated again, up to this many times, until it maps to something new; elites are left alone.  0 = the
  // reference's behaviour: such candidates keep their slot in the population and only a handful of
  // new kernels are measured per generation (6 of 40 on the large tensordot).
  size_t resampleDuplicates = 4;
};

namespace detail {

extern std::atomic<int> tunerSignal; // 0, SIGINT or SIGTERM while a tune() is running

// Statement instances each launched thread executes one after the other, summed over the
// kernels of a mapped TC.
inline double serialDepth(const tc::HipCompilationResult& r) {
  double depth = 0;
  for (const auto& k : r.program.kernels) {
    double points = 0;
    for (const auto& st : k.stages) {
      double p = 1;
      for (const auto& v : st.vars) p *= static_cast<double>(v.extent);
      points += p * static_cast<double>(std::max<size_t>(1, st.stmts.size()));
    }
    double threads = 1;
    for (int a = 0; a < 3; ++a) threads *= static_cast<double>(k.grid[a] * k.block[a]);
    depth += points / std::max(1.0, threads);
  }
  return depth;
}

// `extraSizes`: further extents loops of the TC run over.  The reference derives candidates from
// the input shapes only; the output extents are added here because window-shaped accesses
// (convolutions) loop over sizes that no input extent divides into.
inline std::vector<size_t> inputDivisorsAndPowers2(
    const std::vector<const DLConstTensor*>& inputs, const std::vector<size_t>& extraSizes = {}) {
  std::vector<size_t> sizes = extraSizes;
  for (auto t : inputs) {
    for (int i = 0; i < t->ndim; ++i) sizes.push_back(static_cast<size_t>(t->shape[i]));
  }
  std::sort(sizes.begin(), sizes.end());
  sizes.erase(std::unique(sizes.begin(), sizes.end()), sizes.end());
  std::vector<size_t> out;
  for (auto s : sizes) out = mergeVectors(std::move(out), powers2andCeilDivisors(s));
  // Deviation: exact divisors that cut an extent into at most 16 parts of whole matrix-core steps
  // (multiples of 4, up to 512).  A reduction tile has to divide its extent, and the ceiling
  // divisors of an extent like 1000 (500, 250, 125, 63, ...) hold no tile between 125 and 500.
  std::vector<size_t> exact;
  for (auto s : sizes) {
    for (size_t d = 4; d <= 512 && d <= s; d += 4) {
      if (s % d == 0 && s / d <= 16) exact.push_back(d);
    }
  }
  out = mergeVectors(std::move(out), exact);
  return mergeVectors(std::move(out), powers2andCeilDivisors(256));
}

// Thread counts that cover merged trailing dimensions exactly, whole or in lanes of 2 or 4
// elements (784 = 28*28 -> 196 threads x float4): contiguous dimensions collapse in the mapper, and
// a block that covers the merged extent has no folded points.
inline std::vector<size_t> mergedDimensionThreadCounts(const std::vector<const DLConstTensor*>& inputs) {
  std::vector<size_t> merged;
  for (auto t : inputs) {
    size_t product = 1;
    for (int i = t->ndim - 1; i >= 0 && product <= 4096; --i) {
      product *= static_cast<size_t>(t->shape[i]);
      for (size_t lanes : {1, 2, 4}) {
        if (i < t->ndim - 1 && product % lanes == 0 && product / lanes >= 64 && product / lanes <= 1024) {
          merged.push_back(product / lanes);
        }
      }
    }
  }
  std::sort(merged.begin(), merged.end());
  merged.erase(std::unique(merged.begin(), merged.end()), merged.end());
  return merged;
}

// Random members of generation 0 with informed priors.  A member drawn uniformly from the value
// sets is, for most comprehensions, a kernel of small scalar blocks that loop over what should be
// spread: its tiles, thread counts and grid sizes are independent draws from the divisors of all
// dimensions.  These members are random too, but each draw is coherent with the output's shape:
// some number of trailing output dimensions, taken whole, is spread over the threads (the thread
// count covers their merged extent exactly, in lanes of 1, 2 or 4, or is a plain multiple of the
// wavefront), the dimensions ahead of them get tiles of 1 or a small divisor of their own extent,
// the grid covers the tiles, the unroll budget is large; the remaining switches are coin tosses.
// No family of kernels is named: what the shapes allow is drawn from.
inline std::vector<HipMappingOptions> structuredRandomMembers(
    const HipMappingOptions& base, const std::vector<int64_t>& outShape, size_t count, uint64_t seed) {
  std::vector<HipMappingOptions> members;
  const size_t R = outShape.size();
  if (R == 0 || count == 0) return members;
  std::mt19937_64 rng(seed * 6364136223846793005ULL + 1442695040888963407ULL);
  auto pick = [&](size_t n) { return std::uniform_int_distribution<size_t>(0, n - 1)(rng); };
  auto coin = [&](double p) { return std::bernoulli_distribution(p)(rng); };
  // (threads, lanes, trailing dimensions covered)
  struct Spread {
    uint64_t threads;
    uint32_t lanes;
    size_t dims;
  };
  std::vector<Spread> spreads;
  {
    int64_t merged = 1;
    for (size_t j = R; j-- > 0;) {
      merged *= outShape[j];
      if (merged > 4096) break;
      for (uint32_t lanes : {1u, 2u, 4u}) {
        if (merged % lanes != 0 || outShape[R - 1] % lanes != 0) continue;
        const int64_t t = merged / lanes;
        if (t >= 32 && t <= 1024) spreads.push_back({static_cast<uint64_t>(t), lanes, R - j});
      }
    }
    // plain wavefront multiples over the innermost dimension alone
    for (uint64_t t : {64u, 128u, 256u, 512u}) {
      for (uint32_t lanes : {1u, 2u, 4u}) {
        if (outShape[R - 1] % lanes == 0) spreads.push_back({t, lanes, 1});
      }
    }
  }
  auto smallDivisor = [&](int64_t extent) {
    std::vector<uint64_t> d;
    for (int64_t k = 1; k <= std::min<int64_t>(extent, 32); ++k) {
      if (extent % k == 0) d.push_back(static_cast<uint64_t>(k));
    }
    return d[pick(d.size())];
  };
  const std::vector<FusionStrategy> fusions{FusionStrategy::Max, FusionStrategy::Preserve3Coincident, FusionStrategy::Min};
  for (size_t made = 0, tries = 0; made < count && tries < 20 * count; ++tries) {
    const Spread sp = spreads[pick(spreads.size())];
    const bool rows = coin(0.25); // every output element a reduction of its own along the threads
    HipMappingOptions o = base;
    std::vector<uint64_t> tile, grid;
    const size_t lead = rows ? R : R - std::min(R, sp.dims);
    for (size_t i = 0; i < R; ++i) {
      if (i < lead) {
        const uint64_t t = rows || coin(0.5) ? 1 : smallDivisor(outShape[i]);
        tile.push_back(t);
        if (grid.size() < 3) grid.push_back(static_cast<uint64_t>((outShape[i] + t - 1) / t));
      } else {
        tile.push_back(0);
      }
    }
    if (grid.empty()) grid.push_back(256);
    o.tile(tile);
    o.mapToBlocks(grid);
    o.mapToThreads(std::vector<uint64_t>{rows ? std::vector<uint64_t>{256, 512, 1024}[pick(3)] : sp.threads});
    o.vectorWidth(rows ? std::vector<uint32_t>{1, 4}[pick(2)] : sp.lanes);
    o.unroll(std::vector<uint64_t>{8, 32, 128, 256}[pick(4)]);
    o.matchLibraryCalls(rows || coin(0.2));
    o.useSharedMemory(coin(0.3));
    o.usePrivateMemory(coin(rows ? 0.7 : 0.3));
    o.useReadOnlyCache(coin(0.8));
    o.collapseContiguous(true);
    o.useMfma(!rows && coin(0.15));
    o.prefetchShared(coin(0.2));
    o.outerScheduleFusionStrategy(fusions[pick(3)]);
    o.intraTileScheduleFusionStrategy(fusions[pick(3)]);
    if (std::find(members.begin(), members.end(), o) != members.end()) continue;
    members.push_back(o);
    ++made;
  }
  return members;
}

// Structured starting points next to the caller's base mapping.  The genetic search from one
// point tends to settle in that point's basin (small blocks of scalar accesses for the naive
// options); these cover the three kernel shapes the mapper is built around.  Every value used is
// a member of the search space (0, powers of two up to 256, merged-dimension thread counts).
inline std::vector<HipMappingOptions> heuristicSeeds(
    const HipMappingOptions& base, const std::vector<const DLConstTensor*>& inputs, size_t smallestOutputRank,
    size_t innermostOutputExtent = 0, bool fewOutputs = false, const std::vector<int64_t>& firstOutputShape = {}) {
  std::vector<HipMappingOptions> seeds;
  size_t maxRank = 0;
  uint64_t largest = 256; // largest extent: a grid limit that never forces a block to loop over tiles
  for (auto t : inputs) {
    maxRank = std::max<size_t>(maxRank, t->ndim);
    for (int i = 0; i < t->ndim; ++i) largest = std::max<uint64_t>(largest, static_cast<uint64_t>(t->shape[i]));
  }
  std::vector<uint64_t> threadCounts{256};
  for (size_t m : mergedDimensionThreadCounts(inputs)) {
    if (threadCounts.size() < 3) threadCounts.push_back(m);
  }
  for (uint64_t threads : threadCounts) {
    // streaming: outer dimensions over blocks, a short unrolled dimension, the merged innermost
    // dimension over the threads in lanes of four
    for (uint64_t inner : {1, 4, 8}) {
      HipMappingOptions o = base;
      std::vector<uint64_t> tile{1, inner};
      while (tile.size() < maxRank) tile.push_back(0);
      o.generic.tile(tile);
      o.generic.unroll(128);
      o.mapToThreads(threads).mapToBlocks(largest, 256).useReadOnlyCache(true);
      o.vectorWidthValue = 4;
      o.collapseContiguousValue = true;
      seeds.push_back(o);
    }
    // row reductions: one row per block, the reduction over the threads, later stages of the
    // kernel from the register cache
    for (uint64_t unroll : {8, 64}) {
      HipMappingOptions o = base;
      // the output of lowest rank is what the reductions produce: its dimensions are the rows
      // (tile 1 each: one row per block); the reduction dimensions after them stay whole
      std::vector<uint64_t> rows(std::max<size_t>(1, smallestOutputRank), 1);
      rows.push_back(0);
      o.generic.tile(rows);
      o.generic.unroll(unroll);
      o.generic.matchLibraryCallsValue = true;
      o.generic.outerScheduleOptions.fusionStrategy = FusionStrategy::Max;
      o.mapToThreads(threads).mapToBlocks(largest, 256).useReadOnlyCache(true).usePrivateMemory(true);
      o.vectorWidthValue = 4;
      o.collapseContiguousValue = true;
      seeds.push_back(o);
    }
  }
  // short rows: four of them per block along threadIdx.y, a wavefront each (the results of the
  // reductions then reach the later stages in registers and the block needs no barrier)
  {
    HipMappingOptions o = base;
    std::vector<uint64_t> rows(std::max<size_t>(1, smallestOutputRank), 1);
    rows.back() = 4;
    rows.push_back(0);
    o.generic.tile(rows);
    o.generic.unroll(64);
    o.generic.matchLibraryCallsValue = true;
    o.generic.outerScheduleOptions.fusionStrategy = FusionStrategy::Max;
    o.mapToThreads(64, 4).mapToBlocks(largest, 256).useReadOnlyCache(true).usePrivateMemory(true);
    o.vectorWidthValue = 4;
    o.collapseContiguousValue = true;
    seeds.push_back(o);
  }
  // few outputs, long sums: the rows as above, the outermost reduction index divided among blocks
  // (the slice number is the first variable of the divided statement)
  if (fewOutputs) {
    for (uint32_t slices : {16u, 64u}) {
      HipMappingOptions o = base;
      std::vector<uint64_t> rows(1 + std::max<size_t>(1, smallestOutputRank), 1);
      rows.push_back(0);
      o.generic.tile(rows);
      o.generic.unroll(8);
      o.generic.matchLibraryCallsValue = true;
      o.mapToThreads(256).mapToBlocks(largest, largest, 256).useReadOnlyCache(true);
      o.vectorWidthValue = 4;
      o.collapseContiguousValue = true;
      o.reductionBlocksValue = slices;
      seeds.push_back(o);
    }
  }
  // windows (convolutions with few channels): one image per block with its input window in LDS,
  // the innermost output dimension along threadIdx.x and as many rows as fit along threadIdx.y
  if (innermostOutputExtent >= 8 && innermostOutputExtent <= 256 && smallestOutputRank >= 3) {
    uint64_t rows = 1;
    while (rows * 2 * innermostOutputExtent <= 1024 && rows < 16) rows *= 2;
    for (uint64_t unroll : {4, 16}) {
      HipMappingOptions o = base;
      o.generic.tile(std::vector<uint64_t>{1, 1, 0, 0, 0});
      o.generic.unroll(unroll);
      o.mapToThreads(innermostOutputExtent, rows).mapToBlocks(largest, 256).useSharedMemory(true).useReadOnlyCache(true);
      o.collapseContiguousValue = false;
      seeds.push_back(o);
    }
  }
  // convolutions with many channels on the matrix cores: output (n, m, h, w); one image, 32 (16)
  // output channels and a band of rows per block, the reduction over input channels in tiles of
  // 8 (16) whose input window and weights are staged in LDS
  if (firstOutputShape.size() == 4 && firstOutputShape[2] >= 4) {
    uint64_t band = 1;
    for (uint64_t d = 1; d <= 16; ++d) {
      if (static_cast<uint64_t>(firstOutputShape[2]) % d == 0) band = d;
    }
    for (bool wide : {true, false}) {
      HipMappingOptions o = base;
      o.generic.tile(std::vector<uint64_t>{1, wide ? 32u : 16u, band, 0, wide ? 8u : 16u});
      o.mapToThreads(64, wide ? 8 : 4).mapToBlocks(largest, 256, 256).useSharedMemory(true).useReadOnlyCache(true);
      o.sharedDepth(7);
      o.useMfmaValue = true;
      o.prefetchSharedValue = wide;
      seeds.push_back(o);
    }
  }
  // small batched contractions on the matrix cores: one element of the leading (batch-like)
  // dimensions per block, its whole output tile over four wavefronts, operands through LDS
  if (firstOutputShape.size() >= 3) {
    HipMappingOptions o = base;
    std::vector<uint64_t> tile(firstOutputShape.size(), 0);
    for (size_t i = 0; i < std::max<size_t>(1, firstOutputShape.size() - 3); ++i) tile[i] = 1;
    o.generic.tile(tile);
    o.mapToThreads(64, 4).mapToBlocks(largest, largest).useSharedMemory(true).useReadOnlyCache(true);
    o.useMfmaValue = true;
    seeds.push_back(o);
  }
  // dense contractions on the matrix cores: a 32x32 output tile per block (of one batch element,
  // when the output has more than two dimensions), operands from memory or through LDS
  const bool matrix = firstOutputShape.size() == 2;
  for (bool lds : {false, true}) {
    HipMappingOptions o = base;
    o.generic.tile(matrix ? std::vector<uint64_t>{32, 32} : std::vector<uint64_t>{1, 32, 32});
    o.mapToThreads(64, 4).mapToBlocks(largest, 256).useSharedMemory(lds).useReadOnlyCache(true);
    o.useMfmaValue = true;
    seeds.push_back(o);
  }
  if (matrix) {
    // The reduction extent of a product: an extent two input dimensions have, preferably one the
    // output does not.  Reduction tiles must divide it: the divisor (a multiple of 4, the depth
    // of a matrix-core step) nearest to the wanted tile on a logarithmic scale.
    uint64_t reduction = 0;
    {
      std::map<uint64_t, int> seen;
      for (auto t : inputs) {
        for (int i = 0; i < t->ndim; ++i) ++seen[static_cast<uint64_t>(t->shape[i])];
      }
      bool outside = false;
      for (const auto& e : seen) {
        if (e.second < 2) continue;
        const bool inOutput = static_cast<int64_t>(e.first) == firstOutputShape[0] || static_cast<int64_t>(e.first) == firstOutputShape[1];
        if (!inOutput && !outside) {
          outside = true;
          reduction = 0;
        }
        if (inOutput == !outside) reduction = std::max(reduction, e.first);
      }
    }
    auto reductionTile = [&](uint64_t wanted) -> uint64_t {
      if (reduction == 0 || reduction % wanted == 0) return wanted;
      uint64_t best = 0;
      double bestDistance = 0;
      for (uint64_t d = 4; d <= reduction && d <= 8 * wanted; d += 4) {
        if (reduction % d != 0) continue;
        const double distance = std::fabs(std::log(static_cast<double>(d) / static_cast<double>(wanted)));
        if (best == 0 || distance < bestDistance) {
          best = d;
          bestDistance = distance;
        }
      }
      return best == 0 ? wanted : best;
    };
    // many output tiles: 64x64 per block (128x128 for outputs that fill the device with those),
    // the reduction in tiles of 32 (16) staged through LDS while earlier tiles multiply; four
    // wavefronts, or eight that own rectangles of output tiles
    // (the fourth: 64x128 for outputs with one short side, whose 128x128 tiles are too few)
    for (int variant = 0; variant < 4; ++variant) {
      HipMappingOptions o = base;
      const uint64_t side = variant == 2 ? 128 : 64;
      o.generic.tile(std::vector<uint64_t>{side, variant == 3 ? 128u : side, reductionTile(variant == 2 ? 16 : 32)});
      o.mapToThreads(64, variant == 0 ? 4 : 8).mapToBlocks(largest, largest).useSharedMemory(true).useReadOnlyCache(true);
      o.sharedDepth(7); // (a depth beyond the parallel dimensions: the copies stay inside the reduction tile loop)
      o.useMfmaValue = true;
      o.prefetchSharedValue = true;
      seeds.push_back(o);
    }
    // few output tiles, long reductions: two 16x16 tiles per block of 8 wavefronts, the reduction
    // in tiles of about 256 through two LDS copies
    {
      HipMappingOptions o = base;
      o.generic.tile(std::vector<uint64_t>{16, 32, reductionTile(256)});
      o.mapToThreads(64, 8).mapToBlocks(largest, largest).useSharedMemory(true).useReadOnlyCache(true);
      o.sharedDepth(7);
      o.useMfmaValue = true;
      o.prefetchSharedValue = true;
      seeds.push_back(o);
    }
    // few output tiles: two (one) 16x16 tiles per block of 8 (16) wavefronts, which divide the
    // reduction steps of a tile among themselves
    for (bool two : {true, false}) {
      HipMappingOptions o = base;
      o.generic.tile(std::vector<uint64_t>{16, two ? 32u : 16u});
      o.generic.unroll(256);
      o.mapToThreads(two ? 256 : 512, 2).mapToBlocks(largest, largest).useSharedMemory(true).useReadOnlyCache(true);
      o.useMfmaValue = true;
      o.vectorWidthValue = 2;
      seeds.push_back(o);
    }
  }
  return seeds;
}

// Candidate value sets derived from the input shapes (tc/autotuner/autotuner-inl.h:326-404).
inline TuningConfiguration setupTuningParameters(
    const std::vector<const DLConstTensor*>& inputs, const std::vector<HipMappingOptions>& baseMappings,
    size_t maxUnroll, const std::vector<size_t>& extraSizes = {}) {
  TC_CHECK_GE(inputs.size(), 1u);
  std::vector<size_t> range = inputDivisorsAndPowers2(inputs, extraSizes);
  size_t maxRank = 0;
  for (auto t : inputs) maxRank = std::max<size_t>(maxRank, t->ndim);
  std::vector<size_t> tileRange = range;
  tileRange.push_back(0); // 0 = do not tile this dimension
  std::vector<size_t> blockRange = range, gridRange = range;
  // Deviation: thread counts that cover merged trailing dimensions exactly.
  blockRange = mergeVectors(std::move(blockRange), mergedDimensionThreadCounts(inputs));
  size_t tileDims = maxRank + 2; // (+1 as in the reference, +1 for the slice number of a divided sum)
  for (const auto& b : baseMappings) {
    blockRange = mergeVectors(std::move(blockRange), std::vector<size_t>(b.block.extractVector().begin(), b.block.extractVector().end()));
    gridRange = mergeVectors(std::move(gridRange), std::vector<size_t>(b.grid.extractVector().begin(), b.grid.extractVector().end()));
    tileDims = std::max(tileDims, b.generic.tiling.size());
  }
  TuningConfiguration c;
  c.tilingParams.setRange(1, tileDims, "t", tileRange, "t");
  c.blockParams.setRange(1, 3, "b", blockRange, "b");
  c.gridParams.setRange(1, 3, "g", gridRange, "g");
  c.unrollFactor = RangeParameter(powers2(maxUnroll), "unroll");
  c.privateDepth = RangeParameter({0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10}, "pdepth");
  c.sharedDepth = RangeParameter({0, 1, 2, 3, 4, 5, 6, 7}, "sdepth");
  return c;
}

} // namespace detail

// The reference's form of the cache-file query (tc/autotuner/options_cache-inl.h:337-353): the
// key is derived from the TC text, the entry point and the input tensors.  Empty when the file
// does not exist.
template <typename Backend>
std::vector<typename Backend::MappingOptionsType> loadTopKFromCacheFile(
    const std::string& tc, const std::string& entryPoint, const std::string& cacheFilename,
    const std::vector<const DLConstTensor*>& inputs, size_t count) {
  auto defs = tc::detail::parse(tc);
  TC_CHECK_EQ(defs.count(entryPoint), 1u) << "attempting to access undefined function " << entryPoint;
  CompilerOptions quiet;
  quiet.emitWarnings = false;
  std::ostringstream canon;
  canon << lang::canonicalize(lang::Sema(quiet).checkFunction(defs.at(entryPoint)));
  return loadTopKFromCacheFile<Backend>(
      canon.str(), makeTensorInfoVector(inputs), tc::inferOutputTensorInfo(tc, entryPoint, inputs), cacheFilename, count);
}

template <typename Backend, typename SearchStrategy>
class Autotuner {
 public:
  using ExecutorType = typename Backend::ExecutorType;
  using MappingOptionsType = typename Backend::MappingOptionsType;
  using OptionsCacheType = OptionsCache<Backend>;

  Autotuner() : optionsCache(new OptionsCacheType()) {}

  // `inputs` / `outputs`: device index -> tensors living on that device.  Returns the best
  // topK options found (fewer when not enough candidates were valid).
  std::vector<MappingOptionsType> tune(
      const std::string& tc,
      const std::string& tcEntryPoint,
      const std::unordered_map<size_t, std::vector<const DLConstTensor*>>& inputs,
      std::unordered_map<size_t, std::vector<const DLTensor*>>& outputs,
      const std::vector<MappingOptionsType>& baseMappings,
      size_t topK = 1,
      const TuningParameterFixer& fixedParams = TuningParameterFixer(),
      const TunerSettings& settings = TunerSettings());

  std::shared_ptr<OptionsCacheType> optionsCache;
};

// ------------------------------------------------------------------------------------------
template <typename Backend, typename SearchStrategy>
std::vector<typename Backend::MappingOptionsType> Autotuner<Backend, SearchStrategy>::tune(
    const std::string& tc,
    const std::string& tcEntryPoint,
    const std::unordered_map<size_t, std::vector<const DLConstTensor*>>& inputs,
    std::unordered_map<size_t, std::vector<const DLTensor*>>& outputs,
    const std::vector<MappingOptionsType>& baseMappings,
    size_t topK,
    const TuningParameterFixer& fixedParams,
    const TunerSettings& settings) {
  TC_CHECK(!inputs.empty()) << "no device to tune on";
  TC_CHECK(!baseMappings.empty()) << "need at least one base mapping";
  // every candidate is launched on these tensors
  for (const auto& in : inputs) {
    auto out = outputs.find(in.first);
    TC_CHECK(out != outputs.end()) << "no outputs for device " << in.first;
    Backend::checkTensorsAreLaunchable(in.second, out->second, static_cast<int>(in.first));
  }
  // The device candidates are measured on: the first device of the tuner_devices flag (a comma-
  // separated list, as in the reference, tc/autotuner/autotuner-inl.h:245,279-295) for which
  // tensors were given; the reference spreads candidates over all listed devices, this build
  // measures on one.
  size_t tuningDevice = inputs.begin()->first;
  {
    bool found = false;
    std::stringstream listed(flags().tuner_devices);
    std::string item;
    while (!found && std::getline(listed, item, ',')) {
      if (item.empty()) continue;
      const size_t d = static_cast<size_t>(std::stoul(item));
      if (inputs.count(d)) {
        tuningDevice = d;
        found = true;
      }
    }
    TC_CHECK(found) << "none of the devices of tuner_devices (" << flags().tuner_devices
                    << ") holds the tensors to tune on (device " << inputs.begin()->first << ")";
  }
  auto defs = tc::detail::parse(tc);
  TC_CHECK_EQ(defs.count(tcEntryPoint), 1u) << "attempting to access undefined function " << tcEntryPoint;
  lang::TreeRef tree = defs.at(tcEntryPoint);
  CompilerOptions quiet;
  quiet.emitWarnings = false;
  std::ostringstream canon;
  canon << lang::canonicalize(lang::Sema(quiet).checkFunction(tree));
  const std::string canonicalTc = canon.str();

  const auto& firstInputs = inputs.begin()->second;
  auto inputsInfo = makeTensorInfoVector(firstInputs);
  auto outputsInfo = makeTensorInfoVector(outputs.begin()->second);
  const std::string backendStr = Backend::backendString();

  // search space and starting points
  std::vector<MappingOptionsType> bases = baseMappings;
  if (!settings.cacheFile.empty()) {
    auto restored = loadTopKFromCacheFile<Backend>(
        canonicalTc, inputsInfo, outputsInfo, Backend::makeDeviceFilename(settings.cacheFile), settings.restoreNumber);
    bases.insert(bases.end(), restored.begin(), restored.end());
  }
  std::vector<size_t> outputSizes;
  for (const auto& info : outputsInfo) {
    for (auto e : info.shape) outputSizes.push_back(static_cast<size_t>(e));
  }
  TuningConfiguration space = detail::setupTuningParameters(firstInputs, bases, settings.maxUnroll, outputSizes);
  space.fixParameters(fixedParams);
  if (settings.fixInertParameters) {
    const auto& b0 = bases.front();
    space.fixParametersBeforeScheduling.fixValue(b0.generic.fixParametersBeforeSchedulingValue);
    space.tileImperfectlyNested.fixValue(b0.generic.tileImperfectlyNestedValue);
    space.privateDepth.fixValue(b0.privateDepthValue);
  }
  // Dividing a sum among blocks can only pay where the outputs are too few to fill the device by
  // themselves; elsewhere the gene keeps the base value instead of thinning the search.
  bool fewOutputs = false;
  {
    int64_t fewest = std::numeric_limits<int64_t>::max();
    for (const auto& o : outputsInfo) {
      int64_t n = 1;
      for (auto e : o.shape) n *= e;
      fewest = std::min(fewest, n);
    }
    fewOutputs = fewest < (int64_t(1) << 16);
    if (!fewOutputs) space.reductionBlocks.fixValue(bases.front().reductionBlocksValue);
  }
  std::vector<TuningConfiguration> configs;
  for (const auto& b : bases) {
    TuningConfiguration c = space;
    c.fromHipMappingOptions(b); // throws std::invalid_argument for values outside the space
    configs.push_back(c);
  }
  if (settings.seedHeuristics) {
    // after the caller's own starting points; a seed the (possibly restricted) space cannot
    // express is left out
    size_t smallestOutputRank = outputsInfo.empty() ? 1 : outputsInfo.front().shape.size();
    size_t innermostOutputExtent = 0;
    for (const auto& info : outputsInfo) {
      smallestOutputRank = std::min(smallestOutputRank, info.shape.size());
      if (!info.shape.empty()) innermostOutputExtent = std::max<size_t>(innermostOutputExtent, info.shape.back());
    }
    for (const auto& seed :
         detail::heuristicSeeds(baseMappings.front(), firstInputs, smallestOutputRank, innermostOutputExtent, fewOutputs,
                                outputsInfo.empty() ? std::vector<int64_t>() : outputsInfo.front().shape)) {
      if (std::find(bases.begin(), bases.end(), seed) != bases.end()) continue;
      try {
        TuningConfiguration c = space;
        c.fromHipMappingOptions(seed);
        if (c.isValid()) configs.push_back(c);
      } catch (const std::invalid_argument&) {
      }
    }
  }
  if (settings.structuredRandom && !outputsInfo.empty() && configs.size() < settings.populationSize / 2) {
    // (a member the possibly restricted space cannot express is left out; the rest of the
    // generation is the uniform draw of the search itself)
    const uint64_t drawSeed = settings.seed >= 0 ? static_cast<uint64_t>(settings.seed) : randomSeed();
    for (const auto& member : detail::structuredRandomMembers(
             bases.front(), outputsInfo.front().shape, settings.populationSize / 2 - configs.size(), drawSeed)) {
      try {
        TuningConfiguration c = space;
        c.fromHipMappingOptions(member);
        if (c.isValid()) configs.push_back(c);
      } catch (const std::invalid_argument&) {
      }
    }
  }
  SearchStrategy search(
      configs, settings.generations, settings.populationSize, settings.crossOverRate, settings.mutationRate,
      settings.numberElites, settings.seed);
  const MappingOptionsType baseMapping = bases.front();

  // signals: SIGINT = stop after this generation, SIGTERM = abort now
  detail::tunerSignal = 0;
  auto oldInt = std::signal(SIGINT, [](int s) { detail::tunerSignal = s; });
  auto oldTerm = std::signal(SIGTERM, [](int s) { detail::tunerSignal = s; });
  struct Restore {
    void (*a)(int);
    void (*b)(int);
    ~Restore() {
      std::signal(SIGINT, a);
      std::signal(SIGTERM, b);
    }
  } restore{oldInt, oldTerm};

  Duration bestTime = Duration::max();
  double bestDepth = 0; // serial depth of the candidate that holds bestTime
  // TC_TUNER_TRACE=1: name every candidate before it is compiled and before it is run (finds the
  // one a stalled tuning run is stuck on)
  const char* traceEnv = std::getenv("TC_TUNER_TRACE");
  const bool trace = traceEnv != nullptr && traceEnv[0] != '\0' && traceEnv[0] != '0';
  using Population = std::vector<std::unique_ptr<CandidateConfiguration>>;
  // Different option sets often map to the very same kernels (an option that does not apply to
  // this TC, a tile size beyond an extent, a thread count the mapper tightens): a mapping is
  // compiled and measured once per tuning run, and every later candidate that maps to the same
  // source and launch shapes takes over its result.
  struct Outcome {
    bool done = false, invalid = false;
    Duration runtime = Duration::zero();
  };
  std::map<std::string, std::shared_ptr<Outcome>> outcomes; // guarded by `mu` of the population under evaluation
  size_t duplicates = 0;
  const ir::Function function = tc::detail::translate(tree, firstInputs, quiet);
  tc::detail::checkInputsCompliant(function, firstInputs);
  // compiles (worker threads) and measures (this device) every candidate of `population`;
  // returns the runtimes of the valid ones
  auto mappingKey = [&](const TuningConfiguration& conf) -> std::string { // empty: the mapper refuses it
    try {
      MappingOptionsType options = baseMapping;
      conf.applyToHipMappingOptions(options);
      auto mapped = Backend::compileWithTcMapper(function.name, function, firstInputs, options);
      std::string key = mapped.source;
      for (const auto& k : mapped.kernels) {
        for (int a = 0; a < 3; ++a) key += "|" + std::to_string(k.grid[a]) + "," + std::to_string(k.block[a]);
      }
      return key;
    } catch (const std::exception&) {
      return std::string();
    }
  };
  size_t resampled = 0;
  // bred candidates that would repeat a measured mapping are mutated again (mapping costs a
  // millisecond or two, no JIT)
  auto diversify = [&](Population& population) {
    if (settings.resampleDuplicates == 0) return;
    std::set<std::string> thisGeneration;
    for (size_t i = 0; i < population.size(); ++i) {
      std::string key = mappingKey(population[i]->configuration);
      if (i >= search.numberElites) {
        for (size_t attempt = 0; attempt < settings.resampleDuplicates &&
             (key.empty() || outcomes.count(key) || thisGeneration.count(key));
             ++attempt) {
          search.remutate(*population[i]);
          key = mappingKey(population[i]->configuration);
          ++resampled;
        }
      }
      if (!key.empty()) thisGeneration.insert(key);
    }
  };
  auto evaluatePopulation = [&](Population& population) {
    std::atomic<size_t> cursor{0};
    std::mutex mu;
    std::condition_variable cv;
    struct Job {
      std::unique_ptr<ExecutorType> executor;   // null: failed to compile, or a duplicate
      CandidateConfiguration* candidate = nullptr;
      std::shared_ptr<Outcome> outcome;         // null: failed to compile
      bool duplicate = false;
    };
    std::deque<Job> ready;
    size_t produced = 0;

    auto compileWorker = [&]() {
      for (;;) {
        size_t i = cursor.fetch_add(1);
        if (i >= population.size() || detail::tunerSignal == SIGTERM) return;
        Job job;
        job.candidate = population[i].get();
        try {
          MappingOptionsType options = baseMapping;
          job.candidate->configuration.applyToHipMappingOptions(options);
          if (trace) {
            std::lock_guard<std::mutex> lock(mu);
            std::cerr << "[tuner] " << std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count()
                      << " compiling " << options.toText() << std::endl;
          }
          auto mapped = Backend::compileWithTcMapper(function.name, function, firstInputs, options);
          std::string key = mapped.source;
          for (const auto& k : mapped.kernels) {
            for (int a = 0; a < 3; ++a) key += "|" + std::to_string(k.grid[a]) + "," + std::to_string(k.block[a]);
          }
          {
            std::lock_guard<std::mutex> lock(mu);
            auto found = outcomes.find(key);
            if (found != outcomes.end()) {
              job.outcome = found->second;
              job.duplicate = true;
              ++duplicates;
            } else {
              job.outcome = outcomes.emplace(key, std::make_shared<Outcome>()).first->second;
            }
          }
          if (!job.duplicate) job.executor = tc::detail::makeExecutor<Backend>(function, firstInputs, mapped);
        } catch (const std::exception& e) {
          if (settings.verbose) std::cerr << "[tuner] candidate failed to compile: " << e.what() << std::endl;
          job.executor.reset();
          if (job.outcome && !job.duplicate) {
            std::lock_guard<std::mutex> lock(mu);
            job.outcome->done = job.outcome->invalid = true;
          }
        }
        {
          std::lock_guard<std::mutex> lock(mu);
          ready.push_back(std::move(job));
          ++produced;
        }
        cv.notify_one();
      }
    };

    std::vector<Duration> generationTimes;
    auto evaluate = [&](size_t device) {
      typename Backend::WithDevice guard(device);
      const auto& ins = inputs.at(device);
      const auto& outs = outputs.at(device);
      size_t consumed = 0;
      std::vector<Job> duplicateJobs; // settled once every original of this population has run
      // marks the mapping's outcome when the job goes out of scope, whichever way
      struct Settle {
        Job& job;
        std::mutex& mu;
        ~Settle() {
          if (!job.outcome || job.duplicate) return;
          std::lock_guard<std::mutex> lock(mu);
          job.outcome->done = true;
          job.outcome->invalid = job.candidate->invalid;
          job.outcome->runtime = job.candidate->runtime;
        }
      };
      struct SettleDuplicates {
        std::vector<Job>& jobs;
        ~SettleDuplicates() {
          for (auto& j : jobs) {
            // (an original that never ran, e.g. after an abort, leaves its duplicates invalid)
            j.candidate->invalid = !j.outcome->done || j.outcome->invalid;
            j.candidate->runtime = j.outcome->runtime;
          }
        }
      } settleDuplicates{duplicateJobs};
      while (consumed < population.size()) {
        Job job;
        {
          std::unique_lock<std::mutex> lock(mu);
          cv.wait(lock, [&] { return !ready.empty() || detail::tunerSignal == SIGTERM; });
          if (ready.empty()) return;
          job = std::move(ready.front());
          ready.pop_front();
        }
        ++consumed;
        CandidateConfiguration* cand = job.candidate;
        if (job.duplicate) {
          duplicateJobs.push_back(std::move(job));
          continue;
        }
        Settle settle{job, mu};
        if (!job.executor) {
          cand->invalid = true;
          continue;
        }
        ExecutorType& ex = *job.executor;
        if (trace) {
          MappingOptionsType options = baseMapping;
          cand->configuration.applyToHipMappingOptions(options);
          std::cerr << "[tuner] " << std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count()
                    << " running " << options.toText() << std::endl;
        }
        try {
          // prune launches that cannot fill even one compute unit
          // (the largest launch of the TC counts: a small fill may precede the kernel that matters)
          uint64_t launched = 0;
          for (const auto& kl : ex.compilationResult().kernels) {
            launched = std::max<uint64_t>(launched, uint64_t(kl.grid[0]) * kl.grid[1] * kl.grid[2] * kl.block[0] * kl.block[1] * kl.block[2]);
          }
          if (launched < settings.minLaunchTotalThreads) {
            cand->invalid = true;
            continue;
          }
          // A launch cannot be undone, so a degenerate mapping (a handful of threads walking the
          // whole iteration space) is refused before it is run: statement instances per launched
          // thread, summed over the kernels, against the same figure of the best candidate so far.
          double depth = detail::serialDepth(ex.compilationResult());
          if (bestDepth > 0 && depth > bestDepth * settings.maxSerialDepthRatio) {
            cand->invalid = true;
            continue;
          }
          // first run: stop at once when catastrophically slow (100x), again after warm-up (5x)
          ProfilingInfo first = ex.profile(ins, outs);
          if (bestTime < Duration::max() && first.kernelRuntime >= bestTime * 100) {
            cand->invalid = true;
            continue;
          }
          ProfilingInfo warm = ex.profile(ins, outs);
          if (bestTime < Duration::max() && warm.kernelRuntime >= bestTime * 5) {
            cand->invalid = true;
            continue;
          }
          // Ten samples, the median is the fitness (tc/autotuner/autotuner-inl.h:140-170).  The
          // events around a single launch of a few microseconds see the dispatch path more than the
          // kernel, and the order of short candidates then comes out at random: a sample of a short
          // kernel is the mean over as many back-to-back launches as fill about 200 us (at most 64).
          std::vector<int64_t> runs;
          const int64_t warmNs = std::max<int64_t>(1, warm.kernelRuntime.toNanoSeconds());
          const int repeats = warmNs >= 50000 ? 1 : static_cast<int>(std::min<int64_t>(64, std::max<int64_t>(1, 200000 / warmNs)));
          if (repeats == 1) {
            for (int r = 0; r < 10; ++r) runs.push_back(ex.profile(ins, outs).kernelRuntime.toNanoSeconds());
          } else {
            std::vector<const void*> in;
            std::vector<void*> out;
            for (auto t : ins) in.push_back(static_cast<const char*>(t->data) + t->byte_offset);
            for (auto t : outs) out.push_back(static_cast<char*>(t->data) + t->byte_offset);
            for (int r = 0; r < 10; ++r) runs.push_back(ex.profileRepeated(in, out, repeats).toNanoSeconds() / repeats);
          }
          Duration med = Duration::fromNanoSeconds(median(runs));
          if (med == Duration::zero()) {
            cand->invalid = true;
            continue;
          }
          cand->runtime = med;
          if (med < bestTime) bestDepth = depth;
          bestTime = std::min(bestTime, med, [](Duration a, Duration b) { return a < b; });
          generationTimes.push_back(med);
          MappingOptionsType options = baseMapping;
          cand->configuration.applyToHipMappingOptions(options);
          optionsCache->recordRuntime(canonicalTc, inputsInfo, outputsInfo, backendStr, options, med);
        } catch (const std::exception& e) {
          // a failed launch must not poison later candidates: drain the sticky error state
          tchip_get_last_error();
          if (settings.verbose) std::cerr << "[tuner] candidate failed to run: " << e.what() << std::endl;
          cand->invalid = true;
        }
      }
    };

    std::vector<std::thread> compilers;
    size_t nThreads = std::max<size_t>(1, std::min(settings.threads, population.size()));
    for (size_t t = 0; t < nThreads; ++t) compilers.emplace_back(compileWorker);
    std::thread evaluator(evaluate, tuningDevice);
    for (auto& t : compilers) t.join();
    cv.notify_all();
    evaluator.join();
    if (detail::tunerSignal == SIGTERM) {
      throw std::runtime_error("Abort requested");
    }
    return generationTimes;
  };
  auto report = [&](const std::string& what, std::vector<Duration> generationTimes, size_t size) {
    if (settings.verbose || flags().tuner_gen_log_generations) {
      std::sort(generationTimes.begin(), generationTimes.end());
      std::cerr << "[tuner] " << what << ": " << generationTimes.size() << "/" << size
                << " valid, " << duplicates << " duplicate mappings so far, " << resampled << " mutated again";
      if (!generationTimes.empty()) {
        std::cerr << " (best/median/worst) " << generationTimes.front().toMicroSecondsF() << "/"
                  << generationTimes[generationTimes.size() / 2].toMicroSecondsF() << "/"
                  << generationTimes.back().toMicroSecondsF() << " us";
      }
      std::cerr << std::endl;
    }
  };
  for (size_t gen = 0; gen < settings.generations; ++gen) {
    report("generation " + std::to_string(gen), evaluatePopulation(search.population), search.population.size());
    if (detail::tunerSignal == SIGINT) break;
    if (gen + 1 < settings.generations) {
      search.updateParameters();
      diversify(search.population);
    }
  }
  // Refinement (deviation): the genetic search recombines whole candidates; the last few percent
  // are usually one gene away from its best one.
  {
    const CandidateConfiguration* best = nullptr;
    for (const auto& c : search.population) {
      if (!c->invalid && c->runtime != Duration::zero() && (!best || c->runtime < best->runtime)) best = c.get();
    }
    std::unique_ptr<CandidateConfiguration> center;
    if (best) center.reset(new CandidateConfiguration(*best));
    for (size_t round = 0; center && round < settings.refinementRounds && detail::tunerSignal == 0; ++round) {
      Population neighbours;
      size_t genes = center->configuration.collectParameters().size();
      for (size_t g = 0; g < genes; ++g) {
        for (int step : {-1, 1}) {
          TuningConfiguration c = center->configuration;
          RangeParameter* p = c.collectParameters()[g];
          if (p->isForced()) continue;
          long idx = static_cast<long>(p->selectedIndex()) + step;
          if (idx < 0 || idx >= static_cast<long>(p->numberOptions())) continue;
          p->selectOption(static_cast<size_t>(idx));
          if (c.isValid()) neighbours.emplace_back(new CandidateConfiguration(c));
        }
      }
      if (neighbours.empty()) break;
      report("refinement " + std::to_string(round), evaluatePopulation(neighbours), neighbours.size());
      const CandidateConfiguration* better = nullptr;
      for (const auto& c : neighbours) {
        if (!c->invalid && c->runtime != Duration::zero() && c->runtime < center->runtime &&
            (!better || c->runtime < better->runtime)) {
          better = c.get();
        }
      }
      if (!better) break;
      center.reset(new CandidateConfiguration(*better));
    }
  }
  if (!settings.cacheFile.empty()) {
    appendTopKToCacheFile<Backend>(*optionsCache, Backend::makeDeviceFilename(settings.cacheFile), std::max<size_t>(topK, 10));
  }
  return optionsCache->getTopKOptions(canonicalTc, inputsInfo, outputsInfo, backendStr, topK);
}

} // namespace autotune
} // namespace tc
