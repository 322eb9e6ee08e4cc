// Executor of a TC compiled for the HIP backend (counterpart of
// tc/core/cuda/cuda_tc_executor.h:27-66, cuda_tc_executor.cc:46-149).
#pragma once
#include <memory>

#include "tc/core/hip/hip_backend.h"
#include "tc/core/tc_executor.h"

namespace tc {

class HipTcExecutor : public TcExecutor<HipBackend> {
 public:
  HipTcExecutor(
      const std::vector<TensorInfo>& inputsInfo,
      const std::vector<TensorInfo>& outputsInfo,
      const ir::Function& function,
      const HipCompilationResult& compilationResult);

  void uncheckedRun(
      const std::vector<const void*>& inputs,
      const std::vector<void*>& outputs,
      HipRuntimeInformation info = HipRuntimeInformation()) const override;
  ProfilingInfo profileUnchecked(
      const std::vector<const void*>& inputs,
      const std::vector<void*>& outputs,
      HipRuntimeInformation info = HipRuntimeInformation()) const override;

  // Total device time of `repeats` back-to-back launches (one pair of events around all of
  // them); divide by `repeats` for a per-launch figure that is free of host launch latency.
  Duration profileRepeated(
      const std::vector<const void*>& inputs,
      const std::vector<void*>& outputs,
      int repeats,
      HipRuntimeInformation info = HipRuntimeInformation()) const;

  // Unloads the JIT-compiled module; the executor cannot run afterwards.
  void clearRuntimeCompiledFunction() {
    if (rtcFun_) {
      rtcFun_->clear();
      rtcFun_.reset();
    }
  }
  const HipGrid& grid() const { return result_.grid; }
  const HipBlock& block() const { return result_.block; }
  const HipCompilationResult& compilationResult() const { return result_; }

 private:
  HipCompilationResult result_;
  std::unique_ptr<HipRTCFunction> rtcFun_;
};

} // namespace tc
