// ATen entry points: compile / prepareOutputs / run / profile / uncheckedRun over at::Tensor.
// Signatures of tc/aten/aten_compiler.h:35-92 (implementation: aten_compiler-inl.h:30-86,
// aten_compiler.cc:30-67), on current libtorch.
#pragma once
#include <chrono>
#include <memory>
#include <string>
#include <vector>

#include "tc/aten/aten.h"
#include "tc/core/compiler.h"
#include "tc/core/utils/time.h"

namespace tc {
namespace aten {

// The (contiguous) output shapes as metadata-owning DLTensors without data, as the reference
// returns them (tc/aten/aten_compiler.h:35-38): infos[0]->shape[0], ->ndim, ->dtype.
inline std::vector<tc::DLTensorUPtr> inferOutputTensorInfo(
    const std::string& tc, const std::string& entryPoint, const std::vector<at::Tensor>& inputs) {
  auto in = makeDLConstTensors(inputs);
  std::vector<tc::DLTensorUPtr> out;
  for (const auto& info : tc::inferOutputTensorInfo(tc, entryPoint, extractRawPtrs(in))) {
    out.push_back(makeDLTensor<DLTensor>(info));
  }
  return out;
}

// Uninitialised outputs on the device (and with the options) of inputs[0].
inline std::vector<at::Tensor> prepareOutputs(
    const std::string& tc, const std::string& entryPoint, const std::vector<at::Tensor>& inputs) {
  TC_CHECK_GE(inputs.size(), 1u) << "NYI: Need >0 inputs to determine the backend for the outputs";
  std::vector<at::Tensor> outputs;
  for (const auto& info : inferOutputTensorInfo(tc, entryPoint, inputs)) {
    std::vector<int64_t> shape(info->shape, info->shape + info->ndim);
    outputs.push_back(at::empty(shape, inputs[0].options().dtype(toScalarType(info->dtype))));
  }
  return outputs;
}

template <typename Backend>
std::unique_ptr<typename Backend::ExecutorType> compile(
    const std::string& tc,
    const std::string& entryPoint,
    const std::vector<at::Tensor>& inputs,
    const typename Backend::MappingOptionsType& options,
    const CompilerOptions& compilerOptions = CompilerOptions()) {
  auto in = makeDLConstTensors(inputs);
  return tc::compile<Backend>(tc, entryPoint, extractRawPtrs(in), options, compilerOptions);
}

template <typename Executor>
void run(const Executor& executor, const std::vector<at::Tensor>& inputs, std::vector<at::Tensor>& outputs) {
  auto in = makeDLConstTensors(inputs);
  auto out = makeDLTensors(outputs);
  executor.run(extractRawPtrs(in), extractRawPtrs(out));
}

template <typename Executor>
ProfilingInfo profile(const Executor& executor, const std::vector<at::Tensor>& inputs, std::vector<at::Tensor>& outputs) {
  auto t0 = std::chrono::steady_clock::now();
  auto in = makeDLConstTensors(inputs);
  auto out = makeDLTensors(outputs);
  ProfilingInfo pi = executor.profile(extractRawPtrs(in), extractRawPtrs(out));
  Duration wall = Duration::since(t0);
  pi.cpuOverhead = wall > pi.kernelRuntime ? wall - pi.kernelRuntime : Duration::zero();
  return pi;
}

template <typename Executor>
void uncheckedRun(const Executor& executor, const std::vector<at::Tensor>& inputs, std::vector<at::Tensor>& outputs) {
  std::vector<const void*> in;
  std::vector<void*> out;
  for (const auto& t : inputs) in.push_back(t.data_ptr());
  for (auto& t : outputs) out.push_back(t.data_ptr());
  executor.uncheckedRun(in, out);
}

} // namespace aten
} // namespace tc
