// The reference's second example (tc/examples/blockdiagperm.cc:45-152) on the HIP backend: a
// block-diagonal product followed by a permutation of its columns, written as two comprehensions
// with a reshape in between.  Each is tuned starting from the best options a cache file holds
// (if any), compiled, profiled and run once more unchecked; the tuner's cache is then merged
// back into the file, so that repeated short runs reinforce one another:
//
//   examples/blockdiagperm 3 10 /tmp/blockdiagperm.options
#include <iostream>

#include "tc/aten/aten_autotuner.h"
#include "tc/aten/aten_compiler.h"
#include "tc/autotuner/genetic_search.h"
#include "tc/core/hip/hip_tc_executor.h"

using ATenGeneticHipTuner = tc::aten::ATenAutotuner<tc::HipBackend, tc::autotune::GeneticSearch>;

int main(int argc, char** argv) {
  std::string tc = R"TC(
def blockdiagperm2dfissioned_1(float(B, K, NBYK) I, float(K, NBYK, NBYK) W) -> (O)
{
    O(b, k, nbyk1) +=! I(b, k, r_nbyk0) * W(k, r_nbyk0, nbyk1)
}
def blockdiagperm2dfissioned_2(float(B, N) I, int32(N) Idx) -> (O) {
    O(b, n) = I(b, Idx(n)) where n in 0:N
}
  )TC";
  tc::autotune::TunerSettings settings;
  settings.generations = argc > 1 ? std::stoul(argv[1]) : 3;
  settings.populationSize = argc > 2 ? std::stoul(argv[2]) : 10;
  const std::string optionsCache = argc > 3 ? argv[3] : "";
  auto naive = tc::HipBackend::MappingOptionsType::makeNaiveMappingOptions();

  // 1. The block-diagonal product, starting from the best cached options if there are any.
  auto dev = at::TensorOptions().dtype(at::kFloat).device(at::kCUDA);
  at::Tensor I = at::rand({128, 10, 50}, dev);
  at::Tensor W = at::rand({10, 50, 50}, dev);
  std::vector<tc::HipMappingOptions> options;
  if (!optionsCache.empty()) {
    auto in = tc::aten::makeDLConstTensors({I, W});
    options = tc::autotune::loadTopKFromCacheFile<tc::HipBackend>(
        tc, "blockdiagperm2dfissioned_1", optionsCache, tc::extractRawPtrs(in), 1);
  }
  std::cout << "blockdiagperm2dfissioned_1 starts from " << (options.empty() ? "the naive options" : "cached options") << "\n";
  if (options.empty()) options = {naive};

  ATenGeneticHipTuner geneticAutotuneATen(tc);
  auto bestOption = geneticAutotuneATen.tune("blockdiagperm2dfissioned_1", {I, W}, options, 1, {}, settings);
  TC_CHECK_GT(bestOption.size(), 0u);
  auto pExecutor = tc::aten::compile<tc::HipBackend>(tc, "blockdiagperm2dfissioned_1", {I, W}, bestOption[0]);
  auto outputs = tc::aten::prepareOutputs(tc, "blockdiagperm2dfissioned_1", {I, W});
  auto timings = tc::aten::profile(*pExecutor, {I, W}, outputs);

  // 2. The permutation of the 500 columns of the reshaped result.
  at::Tensor O = outputs[0].clone().resize_({128, 500});
  at::Tensor Idx = at::randperm(500, at::TensorOptions().dtype(at::kInt)).to(at::kCUDA);
  std::vector<tc::HipMappingOptions> options2;
  if (!optionsCache.empty()) {
    auto in = tc::aten::makeDLConstTensors({O, Idx});
    options2 = tc::autotune::loadTopKFromCacheFile<tc::HipBackend>(
        tc, "blockdiagperm2dfissioned_2", optionsCache, tc::extractRawPtrs(in), 1);
  }
  if (options2.empty()) options2 = {naive};
  auto bestOption2 = geneticAutotuneATen.tune("blockdiagperm2dfissioned_2", {O, Idx}, options2, 1, {}, settings);
  TC_CHECK_GT(bestOption2.size(), 0u);
  auto pExecutor2 = tc::aten::compile<tc::HipBackend>(tc, "blockdiagperm2dfissioned_2", {O, Idx}, bestOption2[0]);
  auto outputs2 = tc::aten::prepareOutputs(tc, "blockdiagperm2dfissioned_2", {O, Idx});
  auto timings2 = tc::aten::profile(*pExecutor2, {O, Idx}, outputs2);

  // 3. Best standalone times.
  std::cout << "blockdiagperm2dfissioned_1 size I: " << I.sizes() << ", size W: " << W.sizes()
            << " ran in: " << timings.kernelRuntime.toMicroSecondsF() << "us\n";
  std::cout << "blockdiagperm2dfissioned_2 size O: " << O.sizes() << ", size Idx: " << Idx.sizes()
            << " ran in: " << timings2.kernelRuntime.toMicroSecondsF() << "us\n";

  // 4. Once more without the checks, and against ATen's own routines.
  tc::aten::uncheckedRun(*pExecutor, {I, W}, outputs);
  tc::aten::uncheckedRun(*pExecutor2, {O, Idx}, outputs2);
  at::Tensor product = at::einsum("bkn,knm->bkm", {I, W});
  at::Tensor permuted = at::index_select(O, 1, Idx.to(at::kLong));
  std::cout << "max |diff| of the product vs at::einsum: " << (outputs[0] - product).abs().max().item<float>() << "\n";
  std::cout << "permutation equals at::index_select: " << (at::equal(outputs2[0], permuted) ? "yes" : "no") << "\n";

  // 5. Keep what the tuner found, to start from it next time.
  if (!optionsCache.empty()) {
    tc::autotune::appendTopKToCacheFile(*geneticAutotuneATen.optionsCache, optionsCache, 10);
    std::cout << "best options merged into " << optionsCache << "\n";
  }
  return 0;
}
