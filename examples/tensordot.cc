// The reference's introductory example (tc/examples/tensordot.cc:37-90) on the HIP backend:
// tune a tensordot with the genetic search, compile with the best options, profile, then reuse
// the options on two other shapes.
#include <iostream>

#include "tc/aten/aten_autotuner.h"
#include "tc/aten/aten_compiler.h"
#include "tc/autotuner/genetic_search.h"
#include "tc/core/hip/hip_tc_executor.h"

int main(int argc, char** argv) {
  std::string tc = R"TC(
def tensordot(float(N, C1, C2, H, W) I0,
              float(N, C2, C3, H, W) I1)  -> (O)
{
    O(n, c1, c3, h, w) +=! I0(n, c1, r_c2, h, w) * I1(n, r_c2, c3, h, w)
}
  )TC";
  auto dev = at::TensorOptions().dtype(at::kFloat).device(at::kCUDA);
  at::Tensor I0 = at::rand({16, 8, 16, 17, 25}, dev);
  at::Tensor I1 = at::rand({16, 16, 2, 17, 25}, dev);

  auto naiveOptions = tc::HipBackend::MappingOptionsType::makeNaiveMappingOptions();
  tc::aten::ATenAutotuner<tc::HipBackend, tc::autotune::GeneticSearch> tuner(tc);
  tc::autotune::TunerSettings settings;
  settings.generations = argc > 1 ? std::stoul(argv[1]) : 3;
  settings.populationSize = argc > 2 ? std::stoul(argv[2]) : 10;
  auto bestOption = tuner.tune("tensordot", {I0, I1}, {naiveOptions}, 1, {}, settings);
  TC_CHECK_GT(bestOption.size(), 0u);

  auto pExecutor = tc::aten::compile<tc::HipBackend>(tc, "tensordot", {I0, I1}, bestOption[0]);
  auto outputs = tc::aten::prepareOutputs(tc, "tensordot", {I0, I1});
  auto timings = tc::aten::profile(*pExecutor, {I0, I1}, outputs);
  std::cout << "tensordot size I0: " << I0.sizes() << ", size I1: " << I1.sizes()
            << " ran in: " << timings.kernelRuntime.toMicroSecondsF() << "us\n";
  at::Tensor ref = at::einsum("nachw,ncbhw->nabhw", {I0, I1});
  std::cout << "max |diff| vs at::einsum: " << (outputs[0] - ref).abs().max().item<float>() << "\n";

  for (auto sizes : std::vector<std::pair<std::vector<int64_t>, std::vector<int64_t>>>{
           {{4, 9, 7, 16, 14}, {4, 7, 3, 16, 14}}, {{8, 5, 11, 10, 10}, {8, 11, 16, 10, 10}}}) {
    at::Tensor A = at::rand(sizes.first, dev), B = at::rand(sizes.second, dev);
    auto ex = tc::aten::compile<tc::HipBackend>(tc, "tensordot", {A, B}, bestOption[0]);
    auto outs = tc::aten::prepareOutputs(tc, "tensordot", {A, B});
    auto t = tc::aten::profile(*ex, {A, B}, outs);
    std::cout << "tensordot size I0: " << A.sizes() << ", size I1: " << B.sizes()
              << " ran in: " << t.kernelRuntime.toMicroSecondsF() << "us\n";
  }
  std::cout << tc::HipMappingOptionsAsCpp(bestOption[0]) << std::endl;
  return 0;
}
