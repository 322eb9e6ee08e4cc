// ATenAutotuner: the genetic tuner driven with at::Tensor inputs.
// Interface of tc/aten/aten_autotuner.h:44-90 (implementation: aten_autotuner-inl.h:50-97):
// outputs are prepared here, tuning runs on the device the inputs live on.
#pragma once
#include <string>
#include <vector>

#include "tc/aten/aten_compiler.h"
#include "tc/autotuner/autotuner.h"

namespace tc {
namespace aten {

template <typename Backend, typename Search>
class ATenAutotuner : public tc::autotune::Autotuner<Backend, Search> {
 public:
  using BackendType = Backend;
  using MappingOptionsType = typename BackendType::MappingOptionsType;

  explicit ATenAutotuner(const std::string& tc) : tc_(tc) {}

  std::vector<MappingOptionsType> tune(
      const std::string& tcEntryPoint,
      const std::vector<at::Tensor>& inputs,
      const std::vector<MappingOptionsType>& baseMappings,
      size_t topK = 1,
      const tc::autotune::TuningParameterFixer& fixedParams = tc::autotune::TuningParameterFixer(),
      const tc::autotune::TunerSettings& settings = tc::autotune::TunerSettings()) {
    std::vector<at::Tensor> outputs = prepareOutputs(tc_, tcEntryPoint, inputs);
    auto in = makeDLConstTensors(inputs);
    auto out = makeDLTensors(outputs);
    size_t device = inputs.empty() || !inputs[0].is_cuda() ? 0 : static_cast<size_t>(inputs[0].get_device());
    std::unordered_map<size_t, std::vector<const DLConstTensor*>> inMap;
    std::unordered_map<size_t, std::vector<const DLTensor*>> outMap;
    inMap[device] = extractRawPtrs(in);
    outMap[device] = extractRawPtrs(out);
    return tc::autotune::Autotuner<Backend, Search>::tune(
        tc_, tcEntryPoint, inMap, outMap, baseMappings, topK, fixedParams, settings);
  }

 protected:
  // (kept so that one tuner serves every function of the text; subclasses read it, as in the
  // reference, tc/aten/aten_autotuner.h:86-90)
  const std::string tc_;
};

} // namespace aten
} // namespace tc
