#include "tc/autotuner/parameters.h"

#include <algorithm>
#include <iterator>
#include <sstream>

namespace tc {
namespace autotune {

void RangeParameter::selectFromValue(size_t v) {
  if (fixed_) return;
  auto it = std::find(values_.begin(), values_.end(), v);
  if (it == values_.end()) {
    std::stringstream ss;
    ss << "RangeParameter::selectFromValue: value " << v << " not in range for '" << name
       << "'. The valid values are: ";
    std::copy(values_.begin(), values_.end(), std::ostream_iterator<size_t>(ss, " "));
    throw std::invalid_argument(ss.str());
  }
  selected_ = static_cast<size_t>(it - values_.begin());
}

void MultiRangeParams::setRange(
    size_t minDims, size_t maxDims, const std::string& name, const std::vector<size_t>& values,
    const std::string& dimBaseName) {
  std::vector<size_t> counts;
  for (size_t i = minDims; i <= maxDims; ++i) counts.push_back(i);
  numberDims = RangeParameter(counts, name);
  dims.clear();
  for (size_t i = 0; i < maxDims; ++i) {
    dims.emplace_back(values, dimBaseName + std::to_string(i));
  }
}

void MultiRangeParams::fromValues(const std::vector<uint64_t>& v) {
  numberDims.selectFromValue(v.size());
  for (size_t i = 0; i < v.size() && i < dims.size(); ++i) {
    dims[i].selectFromValue(v[i]);
  }
}

std::vector<uint64_t> MultiRangeParams::toValues() const {
  std::vector<uint64_t> v;
  for (size_t i = 0; i < numberDims.value() && i < dims.size(); ++i) {
    v.push_back(dims[i].value());
  }
  return v;
}

TuningConfiguration::TuningConfiguration()
    : outerFusionStrategy({0, 1, 2}, "fusion strategy"),
      intraTileFusionStrategy({0, 1, 2}, "fusion strategy"),
      fixParametersBeforeScheduling(RangeParameter::boolean("fix parameters before scheduling")),
      unrollFactor({1}, "unroll"),
      tileImperfectlyNested(RangeParameter::boolean("tile imperfectly nested")),
      useSharedMemory(RangeParameter::boolean("use shared memory")),
      usePrivateMemory(RangeParameter::boolean("use private memory")),
      unrollCopyShared(RangeParameter::boolean("unroll copy shared")),
      useReadOnlyCache(RangeParameter::boolean("use readonly cache")),
      matchLibraryCalls(RangeParameter::boolean("match library calls")),
      privateDepth({0}, "pdepth"),
      sharedDepth({0}, "sdepth"),
      vectorWidth({1, 2, 4}, "vector width"),
      collapseContiguous(RangeParameter::boolean("collapse contiguous")),
      useMfma(RangeParameter::boolean("use mfma")),
      prefetchShared(RangeParameter::boolean("prefetch shared")),
      reductionBlocks({1, 2, 4, 8, 16, 32, 64}, "reduction blocks") {
  tilingParams.setRange(1, 1, "t", {0}, "t");
  blockParams.setRange(1, 3, "b", {1}, "b");
  gridParams.setRange(1, 3, "g", {1}, "g");
  // A block is 1..1024 x 1..1024 x 1..64 threads and holds between one and sixteen 64-lane
  // wavefronts (the reference demanded 32..512 threads, tc/autotuner/parameters.cc:357-383).
  addValidator([](const TuningConfiguration& c) {
    size_t b0 = c.blockParams.dims.at(0).value(), b1 = c.blockParams.dims.at(1).value(),
           b2 = c.blockParams.dims.at(2).value();
    if (b0 == 0 || b0 > 1024 || b1 == 0 || b1 > 1024 || b2 == 0 || b2 > 64) return false;
    size_t n = c.blockParams.numberDims.value();
    size_t prod = n == 3 ? b0 * b1 * b2 : n == 2 ? b0 * b1 : b0;
    return prod >= 64 && prod <= 1024;
  });
}

std::vector<RangeParameter*> TuningConfiguration::collectParameters() {
  std::vector<RangeParameter*> p{&outerFusionStrategy, &intraTileFusionStrategy, &fixParametersBeforeScheduling};
  auto multi = [&](MultiRangeParams& m) {
    p.push_back(&m.numberDims);
    for (auto& d : m.dims) p.push_back(&d);
  };
  multi(tilingParams);
  multi(blockParams);
  multi(gridParams);
  for (auto* x : {&unrollFactor, &tileImperfectlyNested, &useSharedMemory, &usePrivateMemory, &unrollCopyShared,
                  &useReadOnlyCache, &matchLibraryCalls, &privateDepth, &sharedDepth, &vectorWidth,
                  &collapseContiguous, &useMfma, &prefetchShared, &reductionBlocks}) {
    p.push_back(x);
  }
  return p;
}

void TuningConfiguration::applyToParameters(const std::function<void(RangeParameter&)>& f) {
  for (auto* p : collectParameters()) f(*p);
}

bool TuningConfiguration::isValid() const {
  for (const auto& v : validators_) {
    if (!v(*this)) return false;
  }
  return true;
}

void TuningConfiguration::fromHipMappingOptions(const HipMappingOptions& o) {
  outerFusionStrategy.selectOption(TuningParameterFixer::toIndex(o.generic.outerScheduleOptions.fusionStrategy));
  intraTileFusionStrategy.selectOption(TuningParameterFixer::toIndex(o.generic.intraTileScheduleOptions.fusionStrategy));
  fixParametersBeforeScheduling.selectFromValue(o.generic.fixParametersBeforeSchedulingValue);
  if (o.generic.hasTiling) tilingParams.fromValues(o.generic.tiling);
  size_t maxUnroll = unrollFactor.values().back();
  unrollFactor.selectFromValue(o.generic.hasUnroll ? std::min<size_t>(o.generic.unrollValue, maxUnroll) : 1);
  tileImperfectlyNested.selectFromValue(o.generic.tileImperfectlyNestedValue);
  matchLibraryCalls.selectFromValue(o.generic.matchLibraryCallsValue);
  blockParams.fromValues(o.block.extractVector());
  gridParams.fromValues(o.grid.extractVector());
  useSharedMemory.selectFromValue(o.useSharedMemoryValue);
  usePrivateMemory.selectFromValue(o.usePrivateMemoryValue);
  unrollCopyShared.selectFromValue(o.unrollCopySharedValue);
  useReadOnlyCache.selectFromValue(o.useReadOnlyCacheValue);
  privateDepth.selectFromValue(o.privateDepthValue);
  sharedDepth.selectFromValue(o.sharedDepthValue);
  vectorWidth.selectFromValue(o.vectorWidthValue);
  collapseContiguous.selectFromValue(o.collapseContiguousValue);
  useMfma.selectFromValue(o.useMfmaValue);
  prefetchShared.selectFromValue(o.prefetchSharedValue);
  size_t blocks = 1; // the largest searched value not above the given one
  for (size_t v : reductionBlocks.values()) {
    if (v <= o.reductionBlocksValue) blocks = std::max(blocks, v);
  }
  reductionBlocks.selectFromValue(blocks);
}

void TuningConfiguration::applyToHipMappingOptions(HipMappingOptions& o) const {
  static const FusionStrategy fs[3] = {FusionStrategy::Max, FusionStrategy::Preserve3Coincident, FusionStrategy::Min};
  o.outerScheduleFusionStrategy(fs[outerFusionStrategy.value()]);
  o.intraTileScheduleFusionStrategy(fs[intraTileFusionStrategy.value()]);
  o.fixParametersBeforeScheduling(fixParametersBeforeScheduling.value());
  o.tile(tilingParams.toValues());
  o.unroll(unrollFactor.value());
  o.tileImperfectlyNested(tileImperfectlyNested.value());
  o.matchLibraryCalls(matchLibraryCalls.value());
  o.mapToThreads(blockParams.toValues());
  o.mapToBlocks(gridParams.toValues());
  o.useSharedMemory(useSharedMemory.value());
  o.usePrivateMemory(usePrivateMemory.value());
  o.unrollCopyShared(unrollCopyShared.value());
  o.useReadOnlyCache(useReadOnlyCache.value());
  o.privateDepth(static_cast<uint32_t>(privateDepth.value()));
  o.sharedDepth(static_cast<uint32_t>(sharedDepth.value()));
  o.vectorWidth(static_cast<uint32_t>(vectorWidth.value()));
  o.collapseContiguous(collapseContiguous.value());
  o.useMfma(useMfma.value());
  o.prefetchShared(prefetchShared.value());
  o.reductionBlocks(static_cast<uint32_t>(reductionBlocks.value()));
}

void TuningConfiguration::fixParameters(const TuningParameterFixer& f) {
  auto fix = [](const TuningParameterFixer::Opt& o, RangeParameter& p) {
    if (o.has) p.fixValue(o.v);
  };
  fix(f.outerFusion_, outerFusionStrategy);
  fix(f.intraFusion_, intraTileFusionStrategy);
  fix(f.fixParams_, fixParametersBeforeScheduling);
  fix(f.unroll_, unrollFactor);
  fix(f.tileImperfect_, tileImperfectlyNested);
  fix(f.useShared_, useSharedMemory);
  fix(f.usePrivate_, usePrivateMemory);
  fix(f.unrollCopy_, unrollCopyShared);
  fix(f.readOnly_, useReadOnlyCache);
  fix(f.matchLib_, matchLibraryCalls);
  fix(f.vector_, vectorWidth);
  fix(f.collapse_, collapseContiguous);
  auto fixMulti = [](bool has, const std::vector<size_t>& v, MultiRangeParams& m) {
    if (!has) return;
    m.numberDims.fixValue(v.size());
    while (m.dims.size() < v.size()) m.dims.emplace_back(std::vector<size_t>{0}, "fixed");
    for (size_t i = 0; i < v.size(); ++i) m.dims[i].fixValue(v[i]);
  };
  fixMulti(f.hasTiling_, f.tiling_, tilingParams);
  fixMulti(f.hasBlock_, f.block_, blockParams);
  fixMulti(f.hasGrid_, f.grid_, gridParams);
}

std::ostream& operator<<(std::ostream& os, const TuningConfiguration& c) {
  HipMappingOptions o = HipMappingOptions::makeNaiveMappingOptions();
  c.applyToHipMappingOptions(o);
  return os << o.toText();
}

} // namespace autotune
} // namespace tc
