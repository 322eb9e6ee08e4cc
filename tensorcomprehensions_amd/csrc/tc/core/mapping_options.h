// Backend-independent mapping options (schedule fusion, tiling, unrolling, library matching).
//
// Names, defaults, presets and the proto2 field numbers follow the reference
// (tc/core/mapping_options.h:92-365, presets tc/core/mapping_options-inl.h:223-262, wire format
// tc/proto/mapping_options.proto:19-72) so tuned option sets can be exchanged as serialized
// strings.  Storage is a plain struct; serialisation is hand-written.
#pragma once
#include <cstdint>
#include <initializer_list>
#include <ostream>
#include <sstream>
#include <string>
#include <vector>

#include "tc/core/check.h"
#include "tc/core/utils/protowire.h"

namespace tc {

enum class FusionStrategy : int { Max = 1, Preserve3Coincident = 2, Min = 3 };

inline std::string toString(FusionStrategy fs) {
  switch (fs) {
    case FusionStrategy::Max: return "Max";
    case FusionStrategy::Preserve3Coincident: return "Preserve3Coincident";
    case FusionStrategy::Min: return "Min";
  }
  return "?";
}
inline bool fusionStrategyFromString(const std::string& s, FusionStrategy* out) {
  if (s == "Max") *out = FusionStrategy::Max;
  else if (s == "Preserve3Coincident") *out = FusionStrategy::Preserve3Coincident;
  else if (s == "Min") *out = FusionStrategy::Min;
  else return false;
  return true;
}
inline std::ostream& operator<<(std::ostream& os, FusionStrategy fs) { return os << toString(fs); }

struct SchedulerOptions {
  FusionStrategy fusionStrategy = FusionStrategy::Preserve3Coincident;
  bool allowSkewing = false;
  bool positiveOrthant = true;
  bool operator==(const SchedulerOptions& o) const {
    return fusionStrategy == o.fusionStrategy && allowSkewing == o.allowSkewing &&
        positiveOrthant == o.positiveOrthant;
  }
  std::string toProto() const {
    protowire::Writer w;
    w.varint(1, static_cast<uint64_t>(fusionStrategy));
    w.boolean(2, allowSkewing);
    w.boolean(3, positiveOrthant);
    return w.str();
  }
  void fromProto(const std::string& s) {
    protowire::Reader r(s);
    while (r.next()) {
      if (r.field() == 1) fusionStrategy = static_cast<FusionStrategy>(r.value());
      if (r.field() == 2) allowSkewing = r.value() != 0;
      if (r.field() == 3) positiveOrthant = r.value() != 0;
    }
  }
};

class MappingOptions {
 public:
  SchedulerOptions outerScheduleOptions, intraTileScheduleOptions;
  bool fixParametersBeforeSchedulingValue = false;
  bool hasTiling = false;
  std::vector<uint64_t> tiling;
  bool hasUnroll = false;
  uint64_t unrollValue = 1;
  bool tileImperfectlyNestedValue = false;
  bool matchLibraryCallsValue = false;

  bool operator==(const MappingOptions& o) const {
    return outerScheduleOptions == o.outerScheduleOptions &&
        intraTileScheduleOptions == o.intraTileScheduleOptions &&
        fixParametersBeforeSchedulingValue == o.fixParametersBeforeSchedulingValue &&
        hasTiling == o.hasTiling && tiling == o.tiling && hasUnroll == o.hasUnroll &&
        (!hasUnroll || unrollValue == o.unrollValue) &&
        tileImperfectlyNestedValue == o.tileImperfectlyNestedValue &&
        matchLibraryCallsValue == o.matchLibraryCallsValue;
  }

  MappingOptions& tile(const std::vector<uint64_t>& sizes) {
    hasTiling = true;
    tiling = sizes;
    return *this;
  }
  MappingOptions& unroll(uint64_t u) {
    hasUnroll = true;
    unrollValue = u;
    return *this;
  }

  std::string toProto() const {
    protowire::Writer w;
    w.bytes(1, outerScheduleOptions.toProto());
    w.bytes(2, intraTileScheduleOptions.toProto());
    w.boolean(3, fixParametersBeforeSchedulingValue);
    if (hasTiling) {
      protowire::Writer t;
      for (auto s : tiling) t.varint(1, s);
      w.bytes(4, t.str());
    }
    if (hasUnroll) w.varint(5, unrollValue);
    w.boolean(6, tileImperfectlyNestedValue);
    w.boolean(7, matchLibraryCallsValue);
    return w.str();
  }
  void fromProto(const std::string& s) {
    protowire::Reader r(s);
    while (r.next()) {
      switch (r.field()) {
        case 1: outerScheduleOptions.fromProto(r.bytes()); break;
        case 2: intraTileScheduleOptions.fromProto(r.bytes()); break;
        case 3: fixParametersBeforeSchedulingValue = r.value() != 0; break;
        case 4: {
          hasTiling = true;
          tiling.clear();
          protowire::Reader t(r.bytes());
          while (t.next()) {
            if (t.field() == 1) t.eachValue([&](uint64_t v) { tiling.push_back(v); });
          }
          break;
        }
        case 5: hasUnroll = true; unrollValue = r.value(); break;
        case 6: tileImperfectlyNestedValue = r.value() != 0; break;
        case 7: matchLibraryCallsValue = r.value() != 0; break;
        default: break;
      }
    }
  }

  // Presets; literal values of tc/core/mapping_options-inl.h:223-262.
  static MappingOptions makeUnmappedMappingOptions() { return MappingOptions(); }
  static MappingOptions makeNaiveMappingOptions() { return MappingOptions().tile({32, 32, 32}).unroll(1); }
  static MappingOptions makeSingleThreadMappingOptions() { return MappingOptions().tile({1}).unroll(1); }
  static MappingOptions makePointwiseMappingOptions() { return MappingOptions().tile({32, 32, 32}).unroll(128); }
  static MappingOptions makeMlpMappingOptions() {
    MappingOptions m;
    m.outerScheduleOptions.fusionStrategy = FusionStrategy::Max;
    return m.tile({1}).unroll(1);
  }
  static MappingOptions makeConvolutionMappingOptions() { return MappingOptions().tile({4, 8, 8, 8}).unroll(1); }
  static MappingOptions makeGroupConvolutionMappingOptions() { return MappingOptions().tile({1, 1}).unroll(1); }
};

// Mixin giving a backend options class (with a `generic` member) the chainable generic setters.
template <typename Derived>
struct GenericOptionsFluent {
  Derived& self() { return static_cast<Derived&>(*this); }
  Derived& tile(const std::vector<uint64_t>& sizes) {
    self().generic.tile(sizes);
    return self();
  }
  Derived& tile(std::initializer_list<uint64_t> sizes) { return tile(std::vector<uint64_t>(sizes)); }
  template <typename... Args>
  Derived& tile(Args... args) {
    return tile(std::vector<uint64_t>{static_cast<uint64_t>(args)...});
  }
  // comma-separated list, e.g. "32,32,4"
  Derived& tile(const std::string& csv) {
    std::vector<uint64_t> v;
    std::stringstream ss(csv);
    std::string item;
    while (std::getline(ss, item, ',')) {
      v.push_back(std::stoull(item));
    }
    return tile(v);
  }
  Derived& unroll(uint64_t u) {
    self().generic.unroll(u);
    return self();
  }
  Derived& fixParametersBeforeScheduling(bool b) {
    self().generic.fixParametersBeforeSchedulingValue = b;
    return self();
  }
  Derived& tileImperfectlyNested(bool b) {
    self().generic.tileImperfectlyNestedValue = b;
    return self();
  }
  Derived& matchLibraryCalls(bool b) {
    self().generic.matchLibraryCallsValue = b;
    return self();
  }
  Derived& scheduleFusionStrategy(FusionStrategy fs) {
    self().generic.outerScheduleOptions.fusionStrategy = fs;
    self().generic.intraTileScheduleOptions.fusionStrategy = fs;
    return self();
  }
  Derived& scheduleFusionStrategy(const std::string& s) {
    FusionStrategy fs;
    TC_CHECK(fusionStrategyFromString(s, &fs)) << "unknown fusion strategy " << s;
    return scheduleFusionStrategy(fs);
  }
  Derived& outerScheduleFusionStrategy(FusionStrategy fs) {
    self().generic.outerScheduleOptions.fusionStrategy = fs;
    return self();
  }
  Derived& outerScheduleFusionStrategy(const std::string& s) {
    FusionStrategy fs;
    TC_CHECK(fusionStrategyFromString(s, &fs)) << "unknown fusion strategy " << s;
    return outerScheduleFusionStrategy(fs);
  }
  Derived& outerScheduleAllowSkewing(bool b) {
    self().generic.outerScheduleOptions.allowSkewing = b;
    return self();
  }
  Derived& outerSchedulePositiveOrthant(bool b) {
    self().generic.outerScheduleOptions.positiveOrthant = b;
    return self();
  }
  Derived& intraTileScheduleFusionStrategy(FusionStrategy fs) {
    self().generic.intraTileScheduleOptions.fusionStrategy = fs;
    return self();
  }
  Derived& intraTileScheduleFusionStrategy(const std::string& s) {
    FusionStrategy fs;
    TC_CHECK(fusionStrategyFromString(s, &fs)) << "unknown fusion strategy " << s;
    return intraTileScheduleFusionStrategy(fs);
  }
  Derived& intraTileScheduleAllowSkewing(bool b) {
    self().generic.intraTileScheduleOptions.allowSkewing = b;
    return self();
  }
  Derived& intraTileSchedulePositiveOrthant(bool b) {
    self().generic.intraTileScheduleOptions.positiveOrthant = b;
    return self();
  }
};

} // namespace tc
