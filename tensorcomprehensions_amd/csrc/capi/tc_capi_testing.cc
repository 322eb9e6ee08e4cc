// libtc_hip_testing.so: what the host-side tests and the sanitized drivers need beyond the product's
// C ABI -- a synthetic genetic search, the whole tune() on a cost model (tc/autotuner/model_backend.h),
// a sample options cache and its self-test.  Test infrastructure: nothing of the product links it.
#include "capi/tc_hip_testing.h"

#include <cstdio>
#include <sstream>

#include "capi/tc_capi_internal.h"
#include "capi/tc_capi_tuner_shared.h"
#include "tc/autotuner/autotuner.h"
#include "tc/autotuner/model_backend.h"
#include "tc/core/hip/hip_tc_executor.h"

namespace {
using namespace tc;
using namespace tc::autotune;
using tc::capi::FakeBackend;
using tc::capi::dumpCache;
using tc::capi::parseSettings;
using tc::capi::readTunerSettings;

// synthetic, deterministic cost of a configuration: distance to a known optimum
double syntheticCost(const TuningConfiguration& c) {
  HipMappingOptions o = HipMappingOptions::makeNaiveMappingOptions();
  c.applyToHipMappingOptions(o);
  double cost = 1.0;
  auto d = [](double a, double b) { return std::abs(std::log2(std::max(a, 1.0)) - std::log2(std::max(b, 1.0))); };
  cost += d(static_cast<double>(o.block[0]), 64) + d(static_cast<double>(o.block[1]), 4);
  cost += d(static_cast<double>(o.grid[0]), 256);
  cost += o.generic.tiling.empty() ? 5 : d(static_cast<double>(o.generic.tiling[0]), 8);
  cost += d(static_cast<double>(o.generic.unrollValue), 16);
  cost += o.useSharedMemoryValue ? 0 : 2;
  cost += o.vectorWidthValue == 4 ? 0 : 1;
  return cost;
}

std::string runSyntheticSearch(const std::map<std::string, std::string>& kv) {
  auto get = [&](const char* k, size_t def) { return kv.count(k) ? static_cast<size_t>(std::stoull(kv.at(k))) : def; };
  int64_t shape0[] = {512, 128}, shape1[] = {128, 256};
  DLConstTensor a{nullptr, {kDLROCM, 0}, 2, {2, 32, 1}, shape0, nullptr, 0};
  DLConstTensor b{nullptr, {kDLROCM, 0}, 2, {2, 32, 1}, shape1, nullptr, 0};
  std::vector<HipMappingOptions> bases{HipMappingOptions::makeNaiveMappingOptions()};
  TuningConfiguration space = tc::autotune::detail::setupTuningParameters({&a, &b}, bases, 256);
  TuningConfiguration start = space;
  start.fromHipMappingOptions(bases[0]);
  GeneticSearch gs({start}, get("generations", 10), get("pop_size", 20), static_cast<uint8_t>(get("crossover_rate", 80)),
                   static_cast<uint8_t>(get("mutation_rate", 7)), get("number_elites", 2),
                   static_cast<int64_t>(get("seed", 1)));
  std::ostringstream out;
  size_t invalidEvery = get("invalid_every", 0);
  for (size_t g = 0; g < gs.numGenerations; ++g) {
    double best = 1e30;
    size_t i = 0;
    for (auto& c : gs.population) {
      TC_CHECK(c->configuration.isValid()) << "search produced an invalid configuration";
      if (invalidEvery && (i++ % invalidEvery) != 0) {
        c->invalid = true;
        continue;
      }
      double cost = syntheticCost(c->configuration);
      c->runtime = Duration::fromMicroSeconds(cost * 10);
      best = std::min(best, cost);
    }
    out << (g ? "," : "") << best;
    TC_CHECK_EQ(gs.population.size(), gs.maxPopulationSize);
    gs.updateParameters();
  }
  return out.str();
}

// The cache the host queries below work on: two TCs, three options for the first one, one of
// them measured three times.
struct SampleCache {
  TensorInfo in0{{2, 32, 1}, 0, {10, 16}, {16, 1}}, in1{{2, 32, 1}, 0, {16, 20}, {20, 1}};
  TensorInfo out0{{2, 32, 1}, 0, {10, 20}, {20, 1}};
  HipMappingOptions o1 = HipMappingOptions::makeNaiveMappingOptions();
  HipMappingOptions o2 = HipMappingOptions::makeNaiveMappingOptions().tile(4, 4).unroll(8);
  HipMappingOptions o3 = HipMappingOptions::makePointwiseMappingOptions();
  OptionsCache<FakeBackend> cache;
  SampleCache() {
    auto us = [](double v) { return Duration::fromMicroSeconds(v); };
    cache.recordRuntime("tcA", {in0, in1}, {out0}, "dev", o1, us(10));
    cache.recordRuntime("tcA", {in0, in1}, {out0}, "dev", o1, us(30));
    cache.recordRuntime("tcA", {in0, in1}, {out0}, "dev", o1, us(20));
    cache.recordRuntime("tcA", {in0, in1}, {out0}, "dev", o2, us(15));
    cache.recordRuntime("tcA", {in0, in1}, {out0}, "dev", o3, us(50));
    cache.recordRuntime("tcB", {in0, in1}, {out0}, "dev", o3, us(5));
  }
};

// The behaviours the reference pins for its compilation cache (test/cuda/test_compilation_cache.cc:
// 133-510: multimap semantics, ranking by the median of all recorded runs, misses, pruning, the
// wire round trip, store / load / append of files) as "name=value" lines for the caller to check.
std::string cacheSelfTest(const std::string& scratch) {
  SampleCache s;
  auto& cache = s.cache;
  std::ostringstream out;
  auto names = [&](const std::vector<std::pair<HipMappingOptions, Duration>>& es) {
    std::string t;
    for (const auto& e : es) {
      t += (t.empty() ? "" : ",") + std::string(e.first == s.o1 ? "o1" : e.first == s.o2 ? "o2" : e.first == s.o3 ? "o3" : "?") +
          "@" + std::to_string(e.second.toNanoSeconds());
    }
    return t;
  };
  out << "size=" << cache.size() << "\n";
  out << "count_tcA=" << cache.count({"tcA", {s.in0, s.in1}, {s.out0}, "dev"}) << "\n";
  out << "keys=" << cache.getKeys().size() << "\n";
  out << "top2_tcA=" << names(cache.getTopKEntries("tcA", {s.in0, s.in1}, {s.out0}, "dev", 2)) << "\n";
  out << "miss_other_tc=" << cache.getTopKOptions("tcC", {s.in0, s.in1}, {s.out0}, "dev", 1).size() << "\n";
  out << "miss_other_sizes=" << cache.getTopKOptions("tcA", {s.in1, s.in0}, {s.out0}, "dev", 1).size() << "\n";
  out << "miss_other_device=" << cache.getTopKOptions("tcA", {s.in0, s.in1}, {s.out0}, "other", 1).size() << "\n";
  TensorInfo misaligned = s.in0;
  misaligned.alignment = 64;
  out << "miss_other_alignment=" << cache.getTopKOptions("tcA", {misaligned, s.in1}, {s.out0}, "dev", 1).size() << "\n";
  out << "retrievals=" << cache.numberAttemptedRetrievals << "," << cache.numberSuccessfulRetrievals << "\n";
  OptionsCache<FakeBackend> copy;
  copy.fromProtobuf(cache.toProtobuf());
  out << "wire_copy_size=" << copy.size() << "\n";
  out << "wire_copy_top3_tcA=" << names(copy.getTopKEntries("tcA", {s.in0, s.in1}, {s.out0}, "dev", 3)) << "\n";
  copy.pruneKeepTopK(1);
  out << "pruned_size=" << copy.size() << "\n";
  out << "pruned_top_tcA=" << names(copy.getTopKEntries("tcA", {s.in0, s.in1}, {s.out0}, "dev", 5)) << "\n";
  if (!scratch.empty()) {
    std::remove(scratch.c_str());
    cache.storeCacheToFile(scratch);
    OptionsCache<FakeBackend> loaded;
    loaded.loadCacheFromFile(scratch);
    out << "file_loaded_size=" << loaded.size() << "\n";
    std::remove(scratch.c_str());
    appendTopKToCacheFile(cache, scratch, 2);
    appendTopKToCacheFile(cache, scratch, 1);
    OptionsCache<FakeBackend> merged;
    merged.loadCacheFromFile(scratch);
    out << "file_appended_size=" << merged.size() << "\n";
    std::remove(scratch.c_str());
  }
  return out.str();
}
} // namespace

extern "C" int tc_testing_query(const char* what, const char* arg, char** out) {
  try {
    std::string w = what ? what : "", a = arg ? arg : "", result;
    if (w == "genetic_search") {
      result = runSyntheticSearch(parseSettings(a.c_str()));
    } else if (w == "tune_on_model") {
      // "<settings>|<entry point>|<shape>;<shape>...|<tc text>": the whole tune() on the host
      // against the cost model of tc/autotuner/model_backend.h (float tensors), from the naive
      // options -> "best=<option text>\ncost_ns=<its modelled time>\nnaive_ns=<that of the naive options>"
      size_t p1 = a.find('|'), p2 = a.find('|', p1 + 1), p3 = a.find('|', p2 + 1);
      TC_CHECK(p1 != std::string::npos && p2 != std::string::npos && p3 != std::string::npos)
          << "expected <settings>|<entry point>|<shapes>|<tc text>";
      tc::autotune::TunerSettings st;
      tc::autotune::TuningParameterFixer fixer;
      size_t topK = 1;
      readTunerSettings(a.substr(0, p1).c_str(), st, fixer, topK);
      const std::string entry = a.substr(p1 + 1, p2 - p1 - 1), text = a.substr(p3 + 1);
      std::vector<std::vector<int64_t>> shapes;
      std::stringstream ss(a.substr(p2 + 1, p3 - p2 - 1));
      std::string sh;
      while (std::getline(ss, sh, ';')) {
        std::vector<int64_t> dims;
        std::stringstream ds(sh);
        std::string d;
        while (std::getline(ds, d, 'x')) dims.push_back(std::stoll(d));
        shapes.push_back(dims);
      }
      std::vector<DLConstTensor> ts(shapes.size());
      std::vector<const DLConstTensor*> ins;
      for (size_t i = 0; i < shapes.size(); ++i) {
        ts[i] = DLConstTensor{nullptr, {kDLROCM, 0}, static_cast<int>(shapes[i].size()), {2, 32, 1}, shapes[i].data(), nullptr, 0};
        ins.push_back(&ts[i]);
      }
      auto infos = tc::inferOutputTensorInfo(text, entry, ins);
      std::vector<DLTensor> os(infos.size());
      std::vector<const DLTensor*> outs;
      for (size_t i = 0; i < infos.size(); ++i) {
        os[i] = DLTensor{nullptr, {kDLROCM, 0}, static_cast<int>(infos[i].shape.size()), infos[i].dtype, infos[i].shape.data(), nullptr, 0};
        outs.push_back(&os[i]);
      }
      using Model = tc::autotune::ModelBackend;
      tc::autotune::Autotuner<Model, tc::autotune::GeneticSearch> tuner;
      std::unordered_map<size_t, std::vector<const DLConstTensor*>> inMap{{0, ins}};
      std::unordered_map<size_t, std::vector<const DLTensor*>> outMap{{0, outs}};
      HipMappingOptions naive = HipMappingOptions::makeNaiveMappingOptions();
      auto best = tuner.tune(text, entry, inMap, outMap, {naive}, topK, fixer, st);
      TC_CHECK(!best.empty()) << "the search found no candidate";
      auto costOf = [&](const HipMappingOptions& o) {
        auto ex = tc::compile<Model>(text, entry, ins, o);
        return ex->profile(ins, outs).kernelRuntime.toNanoSeconds();
      };
      std::ostringstream os2;
      os2 << "best=" << best[0].toText() << "\ncost_ns=" << costOf(best[0]) << "\nnaive_ns=" << costOf(naive);
      result = os2.str();
    } else if (w == "options_cache_selftest") {
      result = cacheSelfTest(a);
    } else if (w == "options_cache_write_sample") {
      SampleCache sample;
      sample.cache.storeCacheToFile(a);
      result = dumpCache(sample.cache);
    } else if (w == "base_outside_space") {
      // a base mapping whose tile size is not a candidate value must be refused
      int64_t shape[] = {10, 16};
      DLConstTensor t{nullptr, {kDLROCM, 0}, 2, {2, 32, 1}, shape, nullptr, 0};
      auto base = HipMappingOptions::makeNaiveMappingOptions().tile(7, 7);
      TuningConfiguration c = tc::autotune::detail::setupTuningParameters({&t}, {base}, 256);
      try {
        c.fromHipMappingOptions(base);
        result = "accepted";
      } catch (const std::invalid_argument& e) {
        result = std::string("invalid_argument: ") + e.what();
      }
    } else {
      TC_CHECK(false) << "unknown testing query '" << w << "'";
    }
    *out = tc::capi::dupString(result);
    return 0;
  } catch (const std::exception& e) {
    tc::capi::lastError = e.what();
    return 1;
  }
}
