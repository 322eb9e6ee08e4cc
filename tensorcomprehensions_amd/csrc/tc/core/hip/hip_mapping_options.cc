#include "tc/core/hip/hip_mapping_options.h"

#include <map>

namespace tc {

namespace {
std::string csv(const std::vector<uint64_t>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) {
    s += (i ? "," : "") + std::to_string(v[i]);
  }
  return s;
}
} // namespace

std::string HipMappingOptions::toText() const {
  std::ostringstream ss;
  ss << "outerScheduleFusionStrategy=" << generic.outerScheduleOptions.fusionStrategy
     << ";outerScheduleAllowSkewing=" << generic.outerScheduleOptions.allowSkewing
     << ";outerSchedulePositiveOrthant=" << generic.outerScheduleOptions.positiveOrthant
     << ";intraTileScheduleFusionStrategy=" << generic.intraTileScheduleOptions.fusionStrategy
     << ";intraTileScheduleAllowSkewing=" << generic.intraTileScheduleOptions.allowSkewing
     << ";intraTileSchedulePositiveOrthant=" << generic.intraTileScheduleOptions.positiveOrthant
     << ";fixParametersBeforeScheduling=" << generic.fixParametersBeforeSchedulingValue;
  if (generic.hasTiling) ss << ";tile=" << csv(generic.tiling);
  if (generic.hasUnroll) ss << ";unroll=" << generic.unrollValue;
  ss << ";tileImperfectlyNested=" << generic.tileImperfectlyNestedValue
     << ";matchLibraryCalls=" << generic.matchLibraryCallsValue
     << ";mapToThreads=" << csv(block.extractVector()) << ";mapToBlocks=" << csv(grid.extractVector())
     << ";useSharedMemory=" << useSharedMemoryValue << ";usePrivateMemory=" << usePrivateMemoryValue
     << ";unrollCopyShared=" << unrollCopySharedValue;
  if (hasMaxSharedMemory) ss << ";maxSharedMemory=" << maxSharedMemoryValue;
  ss << ";useReadOnlyCache=" << useReadOnlyCacheValue;
  if (hasPrivateDepth) ss << ";privateDepth=" << privateDepthValue;
  if (hasSharedDepth) ss << ";sharedDepth=" << sharedDepthValue;
  ss << ";vectorWidth=" << vectorWidthValue << ";collapseContiguous=" << collapseContiguousValue
     << ";useMfma=" << useMfmaValue << ";prefetchShared=" << prefetchSharedValue;
  if (reductionBlocksValue != 1) ss << ";reductionBlocks=" << reductionBlocksValue;
  return ss.str();
}

HipMappingOptions HipMappingOptions::fromText(const std::string& text) {
  HipMappingOptions o = makeNaiveMappingOptions();
  std::stringstream ss(text);
  std::string kv;
  bool first = true;
  while (std::getline(ss, kv, ';')) {
    if (kv.empty()) continue;
    auto eq = kv.find('=');
    std::string k = kv.substr(0, eq), v = eq == std::string::npos ? "" : kv.substr(eq + 1);
    auto b = [&]() { return v == "1" || v == "true" || v == "True"; };
    if (first && eq == std::string::npos) { // leading preset name
      if (k == "naive") o = makeNaiveMappingOptions();
      else if (k == "single_thread") o = makeSingleThreadMappingOptions();
      else if (k == "pointwise") o = makePointwiseMappingOptions();
      else if (k == "mlp") o = makeMlpMappingOptions();
      else if (k == "conv") o = makeConvolutionMappingOptions();
      else if (k == "group_conv") o = makeGroupConvolutionMappingOptions();
      else if (k == "unmapped") o = makeUnmappedMappingOptions();
      else TC_CHECK(false) << "unknown options preset '" << k << "'";
      first = false;
      continue;
    }
    first = false;
    if (k == "outerScheduleFusionStrategy") o.outerScheduleFusionStrategy(v);
    else if (k == "outerScheduleAllowSkewing") o.outerScheduleAllowSkewing(b());
    else if (k == "outerSchedulePositiveOrthant") o.outerSchedulePositiveOrthant(b());
    else if (k == "intraTileScheduleFusionStrategy") o.intraTileScheduleFusionStrategy(v);
    else if (k == "intraTileScheduleAllowSkewing") o.intraTileScheduleAllowSkewing(b());
    else if (k == "intraTileSchedulePositiveOrthant") o.intraTileSchedulePositiveOrthant(b());
    else if (k == "scheduleFusionStrategy") o.scheduleFusionStrategy(v);
    else if (k == "fixParametersBeforeScheduling") o.fixParametersBeforeScheduling(b());
    else if (k == "tile") o.tile(v);
    else if (k == "unroll") o.unroll(std::stoull(v));
    else if (k == "tileImperfectlyNested") o.tileImperfectlyNested(b());
    else if (k == "matchLibraryCalls") o.matchLibraryCalls(b());
    else if (k == "mapToThreads") o.mapToThreads(v);
    else if (k == "mapToBlocks") o.mapToBlocks(v);
    else if (k == "useSharedMemory") o.useSharedMemory(b());
    else if (k == "usePrivateMemory") o.usePrivateMemory(b());
    else if (k == "unrollCopyShared") o.unrollCopyShared(b());
    else if (k == "maxSharedMemory") o.maxSharedMemory(std::stoull(v));
    else if (k == "useReadOnlyCache") o.useReadOnlyCache(b());
    else if (k == "privateDepth") o.privateDepth(static_cast<uint32_t>(std::stoul(v)));
    else if (k == "sharedDepth") o.sharedDepth(static_cast<uint32_t>(std::stoul(v)));
    else if (k == "vectorWidth") o.vectorWidth(static_cast<uint32_t>(std::stoul(v)));
    else if (k == "collapseContiguous") o.collapseContiguous(b());
    else if (k == "useMfma") o.useMfma(b());
    else if (k == "prefetchShared") o.prefetchShared(b());
    else if (k == "reductionBlocks") o.reductionBlocks(static_cast<uint32_t>(std::stoul(v)));
    else TC_CHECK(false) << "unknown mapping option '" << k << "'";
  }
  return o;
}

std::ostream& operator<<(std::ostream& os, const HipMappingOptions& o) {
  return os << o.toText();
}

std::ostream& operator<<(std::ostream& os, const HipMappingOptionsAsCpp& p) {
  const HipMappingOptions& o = p.options;
  std::string in(p.indent + 4, ' ');
  auto bs = [](bool b) { return b ? "true" : "false"; };
  os << std::string(p.indent, ' ') << "tc::HipMappingOptions::makeNaiveMappingOptions()\n"
     << in << ".outerScheduleFusionStrategy(tc::FusionStrategy::" << o.generic.outerScheduleOptions.fusionStrategy << ")\n"
     << in << ".outerScheduleAllowSkewing(" << bs(o.generic.outerScheduleOptions.allowSkewing) << ")\n"
     << in << ".outerSchedulePositiveOrthant(" << bs(o.generic.outerScheduleOptions.positiveOrthant) << ")\n"
     << in << ".intraTileScheduleFusionStrategy(tc::FusionStrategy::" << o.generic.intraTileScheduleOptions.fusionStrategy << ")\n"
     << in << ".intraTileScheduleAllowSkewing(" << bs(o.generic.intraTileScheduleOptions.allowSkewing) << ")\n"
     << in << ".intraTileSchedulePositiveOrthant(" << bs(o.generic.intraTileScheduleOptions.positiveOrthant) << ")\n"
     << in << ".fixParametersBeforeScheduling(" << bs(o.generic.fixParametersBeforeSchedulingValue) << ")\n";
  if (o.generic.hasTiling) {
    os << in << ".tile(";
    for (size_t i = 0; i < o.generic.tiling.size(); ++i) os << (i ? ", " : "") << o.generic.tiling[i];
    os << ")\n";
  }
  if (o.generic.hasUnroll) os << in << ".unroll(" << o.generic.unrollValue << ")\n";
  os << in << ".tileImperfectlyNested(" << bs(o.generic.tileImperfectlyNestedValue) << ")\n"
     << in << ".matchLibraryCalls(" << bs(o.generic.matchLibraryCallsValue) << ")\n"
     << in << ".mapToThreads(" << o.block.toCommaSeparatedString() << ")\n"
     << in << ".mapToBlocks(" << o.grid.toCommaSeparatedString() << ")\n"
     << in << ".useSharedMemory(" << bs(o.useSharedMemoryValue) << ")\n"
     << in << ".usePrivateMemory(" << bs(o.usePrivateMemoryValue) << ")\n"
     << in << ".unrollCopyShared(" << bs(o.unrollCopySharedValue) << ")\n";
  if (o.hasMaxSharedMemory) os << in << ".maxSharedMemory(" << o.maxSharedMemoryValue << ")\n";
  os << in << ".useReadOnlyCache(" << bs(o.useReadOnlyCacheValue) << ")\n";
  if (o.hasPrivateDepth) os << in << ".privateDepth(" << o.privateDepthValue << ")\n";
  if (o.hasSharedDepth) os << in << ".sharedDepth(" << o.sharedDepthValue << ")\n";
  os << in << ".vectorWidth(" << o.vectorWidthValue << ")\n"
     << in << ".collapseContiguous(" << bs(o.collapseContiguousValue) << ")\n"
     << in << ".useMfma(" << bs(o.useMfmaValue) << ")\n"
     << in << ".prefetchShared(" << bs(o.prefetchSharedValue) << ")";
  if (o.reductionBlocksValue != 1) os << "\n" << in << ".reductionBlocks(" << o.reductionBlocksValue << ")";
  return os;
}

} // namespace tc
