// The tuner's search space: one discrete parameter per mapping-option field.
//
// Gene list, order, value sets and the fix-a-gene mechanism follow the reference
// (tc/autotuner/parameters.h:36-236, parameters.cc:100-383).  CDNA4 changes: the block-shape
// validator accepts 64..1024 threads (whole wavefronts up to the device limit) instead of
// 32..512, and three genes are added for the backend's extra options (vector width, collapsing
// of contiguous dimensions).
#pragma once
#include <functional>
#include <ostream>
#include <stdexcept>
#include <string>
#include <vector>

#include "tc/core/hip/hip_mapping_options.h"
#include "tc/core/utils/time.h"

namespace tc {
namespace autotune {

// A parameter that takes one of a fixed list of values; bools are {0, 1}.
class RangeParameter {
 public:
  RangeParameter() = default;
  RangeParameter(std::vector<size_t> values, std::string name) : name(std::move(name)), values_(std::move(values)) {}
  static RangeParameter boolean(const std::string& name) { return RangeParameter({0, 1}, name); }

  size_t numberOptions() const { return fixed_ ? 1 : values_.size(); }
  void selectOption(size_t idx) {
    if (fixed_) return;
    if (idx >= values_.size()) throw std::out_of_range("RangeParameter::selectOption " + name);
    selected_ = idx;
  }
  // throws std::invalid_argument when v is not one of the values
  void selectFromValue(size_t v);
  void fixValue(size_t v) {
    fixed_ = true;
    fixedValue_ = v;
  }
  bool isForced() const { return fixed_; }
  size_t value() const { return fixed_ ? fixedValue_ : values_.at(selected_); }
  size_t selectedIndex() const { return selected_; }
  const std::vector<size_t>& values() const { return values_; }
  std::string name;

 private:
  std::vector<size_t> values_;
  size_t selected_ = 0;
  bool fixed_ = false;
  size_t fixedValue_ = 0;
};

// "number of dimensions" + one value per dimension (tiling, block, grid)
struct MultiRangeParams {
  RangeParameter numberDims;
  std::vector<RangeParameter> dims;
  void setRange(size_t minDims, size_t maxDims, const std::string& name, const std::vector<size_t>& values,
                const std::string& dimBaseName);
  void fromValues(const std::vector<uint64_t>& v);
  std::vector<uint64_t> toValues() const;
};

class TuningParameterFixer;

class TuningConfiguration {
 public:
  TuningConfiguration();

  void fromHipMappingOptions(const HipMappingOptions& o);
  void applyToHipMappingOptions(HipMappingOptions& o) const;

  // all genes in a fixed order
  std::vector<RangeParameter*> collectParameters();
  void applyToParameters(const std::function<void(RangeParameter&)>& f);

  void addValidator(std::function<bool(const TuningConfiguration&)> v) { validators_.push_back(std::move(v)); }
  bool isValid() const;
  void fixParameters(const TuningParameterFixer& fixer);

  RangeParameter outerFusionStrategy, intraTileFusionStrategy; // 0 Max, 1 Preserve3Coincident, 2 Min
  RangeParameter fixParametersBeforeScheduling;
  MultiRangeParams tilingParams, blockParams, gridParams;
  RangeParameter unrollFactor;
  RangeParameter tileImperfectlyNested;
  RangeParameter useSharedMemory, usePrivateMemory, unrollCopyShared, useReadOnlyCache, matchLibraryCalls;
  RangeParameter privateDepth, sharedDepth;
  RangeParameter vectorWidth, collapseContiguous, useMfma, prefetchShared, reductionBlocks;

 private:
  std::vector<std::function<bool(const TuningConfiguration&)>> validators_;
};

std::ostream& operator<<(std::ostream& os, const TuningConfiguration& c);

// Pins chosen genes to a value for the whole search (tc/autotuner/parameters.h:200-236).
class TuningParameterFixer {
 public:
  TuningParameterFixer& fixOuterScheduleFusionStrategy(FusionStrategy fs) { return set(outerFusion_, toIndex(fs)); }
  TuningParameterFixer& fixIntraTileScheduleFusionStrategy(FusionStrategy fs) { return set(intraFusion_, toIndex(fs)); }
  TuningParameterFixer& fixFixParametersBeforeScheduling(bool v) { return set(fixParams_, v); }
  TuningParameterFixer& fixUnrollFactor(size_t v) { return set(unroll_, v); }
  TuningParameterFixer& fixTilingParameters(std::vector<size_t> v) { tiling_ = std::move(v); hasTiling_ = true; return *this; }
  TuningParameterFixer& fixBlockParameters(std::vector<size_t> v) { block_ = std::move(v); hasBlock_ = true; return *this; }
  TuningParameterFixer& fixGridParameters(std::vector<size_t> v) { grid_ = std::move(v); hasGrid_ = true; return *this; }
  TuningParameterFixer& fixTileImperfectlyNested(bool v) { return set(tileImperfect_, v); }
  TuningParameterFixer& fixUseSharedMemory(bool v) { return set(useShared_, v); }
  TuningParameterFixer& fixUsePrivateMemory(bool v) { return set(usePrivate_, v); }
  TuningParameterFixer& fixUnrollCopyShared(bool v) { return set(unrollCopy_, v); }
  TuningParameterFixer& fixUseReadOnlyCache(bool v) { return set(readOnly_, v); }
  TuningParameterFixer& fixMatchLibraryCalls(bool v) { return set(matchLib_, v); }
  TuningParameterFixer& fixVectorWidth(size_t v) { return set(vector_, v); }
  TuningParameterFixer& fixCollapseContiguous(bool v) { return set(collapse_, v); }
  static size_t toIndex(FusionStrategy fs) {
    return fs == FusionStrategy::Max ? 0 : fs == FusionStrategy::Preserve3Coincident ? 1 : 2;
  }

 private:
  struct Opt {
    bool has = false;
    size_t v = 0;
  };
  TuningParameterFixer& set(Opt& o, size_t v) {
    o.has = true;
    o.v = v;
    return *this;
  }
  Opt outerFusion_, intraFusion_, fixParams_, unroll_, tileImperfect_, useShared_, usePrivate_, unrollCopy_,
      readOnly_, matchLib_, vector_, collapse_;
  bool hasTiling_ = false, hasBlock_ = false, hasGrid_ = false;
  std::vector<size_t> tiling_, block_, grid_;
  friend class TuningConfiguration;
};

struct CandidateConfiguration {
  explicit CandidateConfiguration(const TuningConfiguration& c) : configuration(c) {}
  TuningConfiguration configuration;
  Duration runtime = Duration::zero();
  bool invalid = false;
};

} // namespace autotune
} // namespace tc
