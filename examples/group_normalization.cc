// The reference's third example (tc/examples/group_normalization.cc:45-140) on the HIP backend:
// group normalisation with its two reductions and the normalising statement in one
// comprehension, the scale 1 / (D * H * W) written into the text, tuned with the genetic search
// from the naive options or (second argument `best`) from options written with the fluent C++
// builder, then compiled, profiled and compared with at::group_norm.
//
//   examples/group_normalization [generations] [population] [best]
#include <iomanip>
#include <iostream>
#include <sstream>

#include "tc/aten/aten_autotuner.h"
#include "tc/aten/aten_compiler.h"
#include "tc/autotuner/genetic_search.h"
#include "tc/core/hip/hip_tc_executor.h"

// One (n, g) group per block, its 16 x 48 x 48 elements merged into one index that 576 threads
// walk in lanes of four: the normalising statement finds every element in the registers the two
// reductions filled, and the two sums reach it in registers as well.
auto previouslyTunedBestOptions =
    tc::HipMappingOptions::makeNaiveMappingOptions()
        .outerScheduleFusionStrategy(tc::FusionStrategy::Max)
        .outerScheduleAllowSkewing(false)
        .outerSchedulePositiveOrthant(true)
        .intraTileScheduleFusionStrategy(tc::FusionStrategy::Preserve3Coincident)
        .intraTileScheduleAllowSkewing(false)
        .intraTileSchedulePositiveOrthant(true)
        .tile(1, 1, 0)
        .unroll(128)
        .tileImperfectlyNested(false)
        .matchLibraryCalls(true)
        .mapToThreads(576)
        .mapToBlocks(256, 256)
        .useSharedMemory(false)
        .usePrivateMemory(true)
        .unrollCopyShared(false)
        .useReadOnlyCache(true)
        .vectorWidth(4);

int main(int argc, char** argv) {
  std::string tc = R"TC(
def group_normalization(
    float(N, G, D, H, W) I, float(G, D) gamma, float(G, D) beta)
    -> (O, mean, var)
{
    mean(n, g) +=! I(n, g, r_d, r_h, r_w)
     var(n, g) +=! I(n, g, r_d, r_h, r_w) * I(n, g, r_d, r_h, r_w)
    O(n, g, d, h, w) = gamma(g, d)
      * ( I(n, g, d, h, w) - mean(n, g) * <scale> )
      * rsqrt( var(n, g) * <scale>
            - mean(n, g) * mean(n, g) * <scale> * <scale>
            + 1e-5)
      + beta(g, d)
}
  )TC";
  int64_t N = 32, C = 512, G = 32, D = C / G, H = 48, W = 48;
  auto dev = at::TensorOptions().dtype(at::kFloat).device(at::kCUDA);
  at::Tensor I = at::rand({N, G, D, H, W}, dev);
  at::Tensor gamma = at::rand({G, D}, dev);
  at::Tensor beta = at::rand({G, D}, dev);
  // the scale as a literal of the text (nine significant digits: the reference's std::to_string
  // keeps two of them for this size)
  std::ostringstream scale;
  scale << std::setprecision(9) << 1.0f / static_cast<float>(D * H * W);
  for (auto pos = tc.find("<scale>"); pos != std::string::npos; pos = tc.find("<scale>")) {
    tc.replace(pos, std::string("<scale>").size(), scale.str());
  }

  tc::autotune::TunerSettings settings;
  settings.generations = argc > 1 ? std::stoul(argv[1]) : 3;
  settings.populationSize = argc > 2 ? std::stoul(argv[2]) : 10;
  const bool useBestOptions = argc > 3 && std::string(argv[3]) == "best";
  auto baseOptions = useBestOptions ? previouslyTunedBestOptions : tc::HipBackend::MappingOptionsType::makeNaiveMappingOptions();
  tc::aten::ATenAutotuner<tc::HipBackend, tc::autotune::GeneticSearch> geneticAutotuneATen(tc);
  auto bestOption = geneticAutotuneATen.tune("group_normalization", {I, gamma, beta}, {baseOptions}, 1, {}, settings);
  TC_CHECK_GT(bestOption.size(), 0u);

  auto pExecutor = tc::aten::compile<tc::HipBackend>(tc, "group_normalization", {I, gamma, beta}, bestOption[0]);
  auto outputs = tc::aten::prepareOutputs(tc, "group_normalization", {I, gamma, beta});
  auto timings = tc::aten::profile(*pExecutor, {I, gamma, beta}, outputs);
  std::cout << "group_normalization size I: " << I.sizes() << ", ran in: " << timings.kernelRuntime.toMicroSecondsF() << "us\n";
  at::Tensor ref = at::group_norm(I.view({N, C, H, W}), G, gamma.view({C}), beta.view({C}), 1e-5).view({N, G, D, H, W});
  std::cout << "max |diff| vs at::group_norm: " << (outputs[0] - ref).abs().max().item<float>() << "\n";
  std::cout << "best option: " << tc::HipMappingOptionsAsCpp(bestOption[0]) << std::endl;
  return 0;
}
