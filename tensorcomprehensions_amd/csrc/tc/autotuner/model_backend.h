// A backend without a device, for running the tuner's own machinery on the host: the real
// front end and mapper, no JIT, and an executor whose "profile" is a deterministic cost model of
// the mapping (a fixed cost per launch, the statement instances of the busiest thread, a charge
// for every thread a block holds beyond 256 and for LDS).  It knows nothing about the device: it
// only gives the genetic search, the compile/measure pipeline with its threads, the handling of
// duplicate and refused mappings, the refinement rounds and the cache file something to work on
// that behaves alike on every machine, so that they can be tested, also under sanitizers,
// without a GPU.
#pragma once
#include <string>
#include <vector>

#include "tc/autotuner/autotuner.h"
#include "tc/core/hip/hip_backend.h"

namespace tc {
namespace autotune {

class ModelExecutor {
 public:
  ModelExecutor(
      const std::vector<TensorInfo>&, const std::vector<TensorInfo>&, const ir::Function&, const HipCompilationResult& result)
      : result_(result) {}
  const HipCompilationResult& compilationResult() const { return result_; }
  ProfilingInfo profile(const std::vector<const DLConstTensor*>&, const std::vector<const DLTensor*>&) const {
    return ProfilingInfo{Duration::zero(), cost()};
  }
  Duration profileRepeated(const std::vector<const void*>&, const std::vector<void*>&, int repeats) const {
    return cost() * repeats;
  }

 private:
  Duration cost() const {
    double ns = 2500.0 * static_cast<double>(result_.kernels.size()) + 2.0 * detail::serialDepth(result_);
    for (const auto& k : result_.program.kernels) {
      const double threads = static_cast<double>(k.block[0] * k.block[1] * k.block[2]);
      if (threads > 256) ns += 4.0 * (threads - 256);
      ns += static_cast<double>(k.ldsBytes) / 64.0;
    }
    return Duration::fromNanoSeconds(static_cast<int64_t>(ns) + 1);
  }
  HipCompilationResult result_;
};

struct ModelBackend {
  using ExecutorType = ModelExecutor;
  using MappingOptionsType = HipMappingOptions;
  using CompilationResultType = HipCompilationResult;
  struct WithDevice {
    explicit WithDevice(size_t) {}
  };
  static std::string backendString() { return "cost model"; }
  static std::string makeDeviceFilename(const std::string& fn) { return fn + ".model"; }
  static void checkTensorsAreLaunchable(const std::vector<const DLConstTensor*>&, const std::vector<const DLTensor*>&, int = -1) {}
  static CompilationResultType compileWithTcMapper(
      const std::string& name, const ir::Function& f, const std::vector<const DLConstTensor*>& inputs,
      const MappingOptionsType& options) {
    return HipBackend::compileWithTcMapper(name, f, inputs, options);
  }
};

} // namespace autotune
} // namespace tc
