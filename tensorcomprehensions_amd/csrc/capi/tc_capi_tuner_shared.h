// Helpers shared by the tuner's C ABI (tc_capi_tuner.cc) and the testing library (tc_capi_testing.cc).
#pragma once
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "tc/autotuner/autotuner.h"
#include "tc/autotuner/options_cache.h"
#include "tc/core/hip/hip_mapping_options.h"

namespace tc {
namespace capi {

inline std::map<std::string, std::string> parseSettings(const char* s) {
  std::map<std::string, std::string> m;
  if (!s) return m;
  std::stringstream ss(s);
  std::string kv;
  while (std::getline(ss, kv, ';')) {
    auto eq = kv.find('=');
    if (eq != std::string::npos) m[kv.substr(0, eq)] = kv.substr(eq + 1);
  }
  return m;
}

// "key=value;..." -> settings, fixed parameters and the number of results asked for
inline void readTunerSettings(const char* text, tc::autotune::TunerSettings& st, tc::autotune::TuningParameterFixer& fixer, size_t& topK) {
  using namespace tc;
  for (const auto& kv : parseSettings(text)) {
    const std::string &k = kv.first, &v = kv.second;
    auto num = [&]() { return static_cast<size_t>(std::stoull(v)); };
    auto list = [&]() {
      std::vector<size_t> out;
      std::stringstream ss(v);
      std::string item;
      while (std::getline(ss, item, ',')) out.push_back(std::stoull(item));
      return out;
    };
    if (k == "generations") st.generations = num();
    else if (k == "pop_size") st.populationSize = num();
    else if (k == "crossover_rate") st.crossOverRate = static_cast<uint8_t>(num());
    else if (k == "mutation_rate") st.mutationRate = static_cast<uint8_t>(num());
    else if (k == "number_elites") st.numberElites = num();
    else if (k == "threads") st.threads = num();
    else if (k == "seed") st.seed = static_cast<int64_t>(std::stoll(v));
    else if (k == "top_k") topK = num();
    else if (k == "verbose") st.verbose = num() != 0;
    else if (k == "max_unroll") st.maxUnroll = num();
    else if (k == "min_launch_total_threads") st.minLaunchTotalThreads = num();
    else if (k == "max_serial_depth_ratio") st.maxSerialDepthRatio = std::stod(v);
    else if (k == "seed_heuristics") st.seedHeuristics = num() != 0;
    else if (k == "structured_random") st.structuredRandom = num() != 0;
    else if (k == "refinement_rounds") st.refinementRounds = num();
    else if (k == "fix_inert") st.fixInertParameters = num() != 0;
    else if (k == "resample_duplicates") st.resampleDuplicates = num();
    else if (k == "cache_file") st.cacheFile = v;
    else if (k == "fix_tile") fixer.fixTilingParameters(list());
    else if (k == "fix_block") fixer.fixBlockParameters(list());
    else if (k == "fix_grid") fixer.fixGridParameters(list());
    else if (k == "fix_unroll") fixer.fixUnrollFactor(num());
    else if (k == "fix_use_shared_memory") fixer.fixUseSharedMemory(num() != 0);
    else if (k == "fix_match_library_calls") fixer.fixMatchLibraryCalls(num() != 0);
    else if (k == "fix_vector_width") fixer.fixVectorWidth(num());
    else if (k == "fix_collapse_contiguous") fixer.fixCollapseContiguous(num() != 0);
    else if (k == "fix_outer_fusion") {
      FusionStrategy fs;
      TC_CHECK(fusionStrategyFromString(v, &fs)) << "unknown fusion strategy " << v;
      fixer.fixOuterScheduleFusionStrategy(fs);
    } else {
      TC_CHECK(false) << "unknown tuner setting '" << k << "'";
    }
  }
}

// A backend type that only names the options class: for reading cache files of any device.
struct FakeBackend {
  using MappingOptionsType = tc::HipMappingOptions;
  static std::string backendString() { return "fake device"; }
};

// Every entry of a cache as text, one per line: id | backend | inputs | outputs | options | runtimes (ns)
inline std::string dumpCache(const tc::autotune::OptionsCache<FakeBackend>& cache) {
  std::ostringstream ss;
  auto tensors = [&](const std::vector<TensorInfo>& ts) {
    for (size_t i = 0; i < ts.size(); ++i) ss << (i ? ";" : "") << ts[i];
  };
  for (const auto& key : cache.getKeys()) {
    for (const auto& e : cache.getTopKEntries(key.id, key.inputs, key.outputs, key.backendStr, 1000)) {
      ss << key.id << " | " << key.backendStr << " | ";
      tensors(key.inputs);
      ss << " | ";
      tensors(key.outputs);
      ss << " | " << e.first.toText() << " | median " << e.second.toNanoSeconds() << "\n";
    }
  }
  return ss.str();
}

} // namespace capi
} // namespace tc
