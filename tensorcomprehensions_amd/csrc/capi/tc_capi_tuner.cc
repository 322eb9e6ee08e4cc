// tc_autotune: C ABI of the genetic autotuner.
#include "tc/core/mapper/sync_placement.h"
#include <cstdio>
#include <sstream>

#include "capi/tc_capi_internal.h"
#include "tc/autotuner/autotuner.h"
#include "capi/tc_capi_tuner_shared.h"
#include "tc/core/hip/hip_tc_executor.h"


extern "C" int tc_autotune(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    const tc_dl_tensor* const* outputs, int numOutputs, const char* baseOptions, const char* settingsText,
    char** best) {
  using namespace tc;
  try {
    autotune::TunerSettings st;
    autotune::TuningParameterFixer fixer;
    size_t topK = 1;
    tc::capi::readTunerSettings(settingsText, st, fixer, topK);
    // base options: one per line
    std::vector<HipMappingOptions> bases;
    std::stringstream bs(baseOptions ? baseOptions : "naive");
    std::string line;
    while (std::getline(bs, line)) {
      if (!line.empty()) bases.push_back(HipMappingOptions::fromText(line));
    }
    // (tune() refuses host memory and null data before anything is launched; this call orders
    // that check ahead of the first HIP call, so it also works on a machine without a GPU)
    HipBackend::checkTensorsAreLaunchable(capi::constTensors(inputs, numInputs), capi::mutTensors(outputs, numOutputs));
    int dev = 0;
    TC_HIP_CHECK(tchip_get_device(&dev));
    std::unordered_map<size_t, std::vector<const DLConstTensor*>> in;
    std::unordered_map<size_t, std::vector<const DLTensor*>> out;
    in[dev] = capi::constTensors(inputs, numInputs);
    out[dev] = capi::mutTensors(outputs, numOutputs);
    autotune::Autotuner<HipBackend, autotune::GeneticSearch> tuner;
    auto result = tuner.tune(tcText, entry, in, out, bases, topK, fixer, st);
    std::string text;
    for (const auto& o : result) text += o.toText() + "\n";
    *best = capi::dupString(text);
    return 0;
  } catch (const std::exception& e) {
    tc::capi::lastError = e.what();
    return 1;
  }
}

extern "C" int tc_options_cache_load(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    const char* cacheFile, int count, char** best) {
  using namespace tc;
  try {
    auto defs = tc::detail::parse(tcText);
    TC_CHECK_EQ(defs.count(entry), 1u) << "attempting to access undefined function " << entry;
    CompilerOptions quiet;
    quiet.emitWarnings = false;
    std::ostringstream canon;
    canon << lang::canonicalize(lang::Sema(quiet).checkFunction(defs.at(entry)));
    auto in = capi::constTensors(inputs, numInputs);
    auto inputsInfo = makeTensorInfoVector(in);
    auto outputsInfo = tc::inferOutputTensorInfo(tcText, entry, in);
    auto found = autotune::loadTopKFromCacheFile<HipBackend>(
        canon.str(), inputsInfo, outputsInfo, HipBackend::makeDeviceFilename(cacheFile), static_cast<size_t>(std::max(count, 0)));
    std::string text;
    for (const auto& o : found) text += o.toText() + "\n";
    *best = capi::dupString(text);
    return 0;
  } catch (const std::exception& e) {
    tc::capi::lastError = e.what();
    return 1;
  }
}

// ------------------------------------------------------------------------------------------
// tc_host_query: tuner logic that needs no device
// ------------------------------------------------------------------------------------------
namespace {
using namespace tc;
using namespace tc::autotune;
using tc::capi::FakeBackend;
using tc::capi::dumpCache;

std::string joinSizes(const std::vector<size_t>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + std::to_string(v[i]);
  return s;
}



} // namespace

extern "C" int tc_host_query(const char* what, const char* arg, char** out) {
  try {
    std::string w = what, a = arg ? arg : "";
    std::string result;
    if (w == "powers2_and_ceil_divisors") {
      result = joinSizes(powers2andCeilDivisors(std::stoull(a)));
    } else if (w == "median") {
      std::vector<long long> v;
      std::stringstream ss(a);
      std::string item;
      while (std::getline(ss, item, ',')) v.push_back(std::stoll(item));
      result = std::to_string(median(v));
    } else if (w == "search_space") {
      std::vector<std::vector<int64_t>> shapes;
      std::stringstream ss(a);
      std::string sh;
      while (std::getline(ss, sh, ';')) {
        std::vector<int64_t> dims;
        std::stringstream ds(sh);
        std::string d;
        while (std::getline(ds, d, 'x')) dims.push_back(std::stoll(d));
        shapes.push_back(dims);
      }
      std::vector<DLConstTensor> ts(shapes.size());
      std::vector<const DLConstTensor*> ptrs;
      for (size_t i = 0; i < shapes.size(); ++i) {
        ts[i] = DLConstTensor{nullptr, {kDLROCM, 0}, static_cast<int>(shapes[i].size()), {2, 32, 1}, shapes[i].data(), nullptr, 0};
        ptrs.push_back(&ts[i]);
      }
      TuningConfiguration c = tc::autotune::detail::setupTuningParameters(ptrs, {HipMappingOptions::makeNaiveMappingOptions()}, 256);
      result = "tile_dims=" + std::to_string(c.tilingParams.dims.size()) + ";tile=" + joinSizes(c.tilingParams.dims[0].values()) +
          ";block=" + joinSizes(c.blockParams.dims[0].values()) + ";grid=" + joinSizes(c.gridParams.dims[0].values()) +
          ";unroll=" + joinSizes(c.unrollFactor.values()) + ";genes=" + std::to_string(c.collectParameters().size());
    } else if (w == "tuner_seeds") {
      // "rank[,innermost output extent]:shapes", shapes as for search_space -> the structured
      // starting points the search space accepts (one option text per line), as generation 0
      // would hold them next to the naive options
      std::vector<std::vector<int64_t>> shapes;
      size_t colon = a.find(':');
      TC_CHECK(colon != std::string::npos) << "expected <smallest output rank>[,<innermost output extent>[,<first output shape>]]:<shapes>";
      std::string head = a.substr(0, colon);
      size_t comma = head.find(',');
      size_t smallestOutputRank = std::stoul(head.substr(0, comma));
      size_t innermostOutputExtent = comma == std::string::npos ? 0 : std::stoul(head.substr(comma + 1));
      std::vector<int64_t> firstOutputShape;
      size_t second = comma == std::string::npos ? std::string::npos : head.find(',', comma + 1);
      if (second != std::string::npos) {
        std::stringstream os(head.substr(second + 1));
        std::string d;
        while (std::getline(os, d, 'x')) firstOutputShape.push_back(std::stoll(d));
      }
      std::stringstream ss(a.substr(colon + 1));
      std::string sh;
      while (std::getline(ss, sh, ';')) {
        std::vector<int64_t> dims;
        std::stringstream ds(sh);
        std::string d;
        while (std::getline(ds, d, 'x')) dims.push_back(std::stoll(d));
        shapes.push_back(dims);
      }
      std::vector<DLConstTensor> ts(shapes.size());
      std::vector<const DLConstTensor*> ptrs;
      for (size_t i = 0; i < shapes.size(); ++i) {
        ts[i] = DLConstTensor{nullptr, {kDLROCM, 0}, static_cast<int>(shapes[i].size()), {2, 32, 1}, shapes[i].data(), nullptr, 0};
        ptrs.push_back(&ts[i]);
      }
      HipMappingOptions naive = HipMappingOptions::makeNaiveMappingOptions();
      std::vector<size_t> outputSizes;
      if (innermostOutputExtent > 0) outputSizes.push_back(innermostOutputExtent);
      TuningConfiguration space = tc::autotune::detail::setupTuningParameters(ptrs, {naive}, 256, outputSizes);
      for (const auto& seed : tc::autotune::detail::heuristicSeeds(naive, ptrs, smallestOutputRank, innermostOutputExtent, false, firstOutputShape)) {
        try {
          TuningConfiguration c = space;
          c.fromHipMappingOptions(seed);
          if (!c.isValid()) continue;
          HipMappingOptions applied = naive;
          c.applyToHipMappingOptions(applied);
          result += (result.empty() ? "" : "\n") + applied.toText();
        } catch (const std::invalid_argument&) {
        }
      }
    } else if (w == "sync_placement") {
      // "cyclic;n;i:k:level,i:k:level,..." -> "position:level,..." (barrier after child `position`)
      std::stringstream ss(a);
      std::string cyc, num, triples, item;
      std::getline(ss, cyc, ';');
      std::getline(ss, num, ';');
      std::getline(ss, triples, ';');
      int n = std::stoi(num);
      tc::mapper::SyncNeeds need(n, std::vector<int>(n, 0));
      std::stringstream ts(triples);
      while (std::getline(ts, item, ',')) {
        int i = 0, k = 0, lev = 0;
        TC_CHECK(std::sscanf(item.c_str(), "%d:%d:%d", &i, &k, &lev) == 3) << "bad requirement '" << item << "'";
        TC_CHECK(i >= 0 && i < n && k >= 0 && k < n && lev >= 0 && lev <= 2) << "requirement out of range";
        need[i][k] = lev;
      }
      auto syncs = tc::mapper::findBestSyncs(need, cyc == "1");
      TC_CHECK(tc::mapper::syncsAreSufficient(need, cyc == "1", syncs)) << "placement misses a requirement";
      for (const auto& sy : syncs) {
        result += (result.empty() ? "" : ",") + std::to_string(sy.first) + ":" + std::to_string(static_cast<int>(sy.second));
      }
    } else if (w == "options_cache_dump") {
      OptionsCache<FakeBackend> loaded;
      loaded.loadCacheFromFile(a);
      result = dumpCache(loaded);
    } else {
      TC_CHECK(false) << "unknown host query '" << w << "'";
    }
    *out = tc::capi::dupString(result);
    return 0;
  } catch (const std::exception& e) {
    tc::capi::lastError = e.what();
    return 1;
  }
}
