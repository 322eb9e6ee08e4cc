// Compile-only check of the ATen-level boundary: the call shapes a user of the reference writes
// (tc/aten/aten_compiler.h:35-92, tc/aten/aten_autotuner.h:44-90) must compile unchanged with
// tc::HipBackend in place of tc::CudaBackend.  Nothing here runs on a device.
#include <string>
#include <vector>

#include "tc/aten/aten_autotuner.h"
#include "tc/aten/aten_compiler.h"
#include "tc/autotuner/genetic_search.h"
#include "tc/core/hip/hip_backend.h"
#include "tc/core/hip/hip_tc_executor.h"

namespace {

// a subclass reads the TC text the tuner was built from, as the reference's tests do
class NamedTuner : public tc::aten::ATenAutotuner<tc::HipBackend, tc::autotune::GeneticSearch> {
 public:
  using Base = tc::aten::ATenAutotuner<tc::HipBackend, tc::autotune::GeneticSearch>;
  static_assert(std::is_same<Base::BackendType, tc::HipBackend>::value, "BackendType");
  static_assert(std::is_same<Base::MappingOptionsType, tc::HipMappingOptions>::value, "MappingOptionsType");
  explicit NamedTuner(const std::string& tc) : Base(tc) {}
  size_t textLength() const { return tc_.size(); }
};

int64_t useTheBoundary(const std::string& tc, const std::vector<at::Tensor>& inputs) {
  // metadata-owning DLTensors: infos[0]->shape[0]
  std::vector<tc::DLTensorUPtr> infos = tc::aten::inferOutputTensorInfo(tc, "f", inputs);
  int64_t first = infos.empty() || infos[0]->ndim == 0 ? 0 : infos[0]->shape[0];
  std::vector<at::Tensor> outputs = tc::aten::prepareOutputs(tc, "f", inputs);
  auto pExecutor = tc::aten::compile<tc::HipBackend>(tc, "f", inputs, tc::HipMappingOptions::makeNaiveMappingOptions());
  tc::aten::run(*pExecutor, inputs, outputs);
  tc::ProfilingInfo info = tc::aten::profile(*pExecutor, inputs, outputs);
  (void)info;
  tc::aten::uncheckedRun(*pExecutor, inputs, outputs);
  NamedTuner tuner(tc);
  std::vector<tc::HipMappingOptions> best =
      tuner.tune("f", inputs, {tc::HipMappingOptions::makeNaiveMappingOptions()}, 1, tc::autotune::TuningParameterFixer());
  return first + static_cast<int64_t>(best.size() + tuner.textLength());
}

} // namespace

int main() {
  (void)&useTheBoundary;
  return 0;
}
