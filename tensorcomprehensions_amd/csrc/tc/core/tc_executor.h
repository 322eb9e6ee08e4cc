// Backend-generic executor: owns the metadata a compiled TC was specialised on, checks run-time
// tensors against it and forwards to the backend's launch.  Counterpart of
// tc/core/tc_executor.h:67-121 and tc/core/tc_executor-inl.h:33-154.
#pragma once
#include <chrono>
#include <sstream>
#include <string>
#include <vector>

#include "tc/core/check.h"
#include "tc/core/ir.h"
#include "tc/core/tensor.h"
#include "tc/core/utils/time.h"
#include "tc/lang/tree.h"

namespace tc {

namespace detail {
// Count, rank, dtype and shape must match what was compiled; strides are not compared
// (tc/core/tc_executor-inl.h:33-67).
template <typename DLT>
void checkSizesAndStridesAreCompliant(
    const std::vector<const DLT*>& actual, const std::vector<TensorInfo>& expected, const char* what) {
  TC_CHECK_EQ(actual.size(), expected.size()) << "wrong number of " << what << " tensors";
  for (size_t i = 0; i < actual.size(); ++i) {
    const DLT* t = actual[i];
    const TensorInfo& e = expected[i];
    TC_CHECK_EQ(static_cast<size_t>(t->ndim), e.shape.size())
        << what << " " << i << ": expected " << e.shape.size() << " dimensions but found tensor with " << t->ndim
        << " dimensions";
    TC_CHECK(t->dtype.code == e.dtype.code && t->dtype.bits == e.dtype.bits)
        << what << " " << i << ": expected " << toString(e.dtype) << " but found " << toString(t->dtype);
    for (int d = 0; d < t->ndim; ++d) {
      TC_CHECK_EQ(t->shape[d], e.shape[d]) << what << " " << i << " dimension " << d << ": size differs from the compiled one";
    }
    // Generated kernels index tensors as dense row-major arrays (as the reference's do,
    // tc/core/polyhedral/cuda/codegen.cc:200-243, where a strided view silently computes on the
    // wrong elements); a tensor whose strides say otherwise is refused instead.
    if (t->strides) {
      int64_t expect = 1;
      for (int d = t->ndim - 1; d >= 0; --d) {
        if (t->shape[d] != 1 && t->strides[d] != expect) {
          std::stringstream ss;
          ss << what << " " << i << " is not contiguous: " << *t;
          throw InvalidStrideException(ss.str());
        }
        expect *= t->shape[d];
      }
    }
  }
}
} // namespace detail

template <typename Backend>
class TcExecutor {
 protected:
  TcExecutor(
      std::vector<TensorInfo> inputsInfo,
      std::vector<TensorInfo> outputsInfo,
      const ir::Function& function,
      const typename Backend::CompilationResultType& compilationResult)
      : compiledSource(compilationResult.source),
        inputsInfo_(std::move(inputsInfo)),
        outputsInfo_(std::move(outputsInfo)),
        function_(function) {}

 public:
  virtual ~TcExecutor() {}
  TcExecutor(TcExecutor&&) = delete;
  TcExecutor& operator=(TcExecutor&&) = delete;
  TcExecutor(const TcExecutor&) = delete;
  TcExecutor& operator=(const TcExecutor&) = delete;

  // Checked run; the tensors are borrowed for the duration of the call.  May be called
  // repeatedly with different base pointers of identical shapes.  Does not synchronise.
  // Beyond the reference's checks the backend also refuses tensors a kernel must not be
  // launched on (host memory, null data, another device): the reference launches on them.
  void run(
      const std::vector<const DLConstTensor*>& inputs,
      const std::vector<const DLTensor*>& outputs,
      typename Backend::RuntimeInformation info = typename Backend::RuntimeInformation()) const {
    detail::checkSizesAndStridesAreCompliant(inputs, inputsInfo_, "input");
    detail::checkSizesAndStridesAreCompliant(outputs, outputsInfo_, "output");
    Backend::checkTensorsAreLaunchable(inputs, outputs);
    std::vector<const void*> in;
    std::vector<void*> out;
    for (auto t : inputs) in.push_back(static_cast<const char*>(t->data) + t->byte_offset);
    for (auto t : outputs) out.push_back(static_cast<char*>(t->data) + t->byte_offset);
    uncheckedRun(in, out, info);
  }

  // Checked run bracketed by device events; synchronises.  cpuOverhead = wall clock - kernel.
  ProfilingInfo profile(
      const std::vector<const DLConstTensor*>& inputs,
      const std::vector<const DLTensor*>& outputs,
      typename Backend::RuntimeInformation info = typename Backend::RuntimeInformation()) const {
    auto t0 = std::chrono::steady_clock::now();
    detail::checkSizesAndStridesAreCompliant(inputs, inputsInfo_, "input");
    detail::checkSizesAndStridesAreCompliant(outputs, outputsInfo_, "output");
    Backend::checkTensorsAreLaunchable(inputs, outputs);
    std::vector<const void*> in;
    std::vector<void*> out;
    for (auto t : inputs) in.push_back(static_cast<const char*>(t->data) + t->byte_offset);
    for (auto t : outputs) out.push_back(static_cast<char*>(t->data) + t->byte_offset);
    ProfilingInfo pi = profileUnchecked(in, out, info);
    Duration wall = Duration::since(t0);
    pi.cpuOverhead = wall > pi.kernelRuntime ? wall - pi.kernelRuntime : Duration::zero();
    return pi;
  }

  virtual void uncheckedRun(
      const std::vector<const void*>& inputs,
      const std::vector<void*>& outputs,
      typename Backend::RuntimeInformation info = typename Backend::RuntimeInformation()) const = 0;
  virtual ProfilingInfo profileUnchecked(
      const std::vector<const void*>& inputs,
      const std::vector<void*>& outputs,
      typename Backend::RuntimeInformation info = typename Backend::RuntimeInformation()) const = 0;

  const std::vector<TensorInfo>& inputsInfo() const { return inputsInfo_; }
  const std::vector<TensorInfo>& outputsInfo() const { return outputsInfo_; }
  const ir::Function& function() const { return function_; }

  const std::string compiledSource;

 protected:
  std::vector<TensorInfo> inputsInfo_;
  std::vector<TensorInfo> outputsInfo_;
  ir::Function function_;
};

} // namespace tc
