// Backend-generic compile pipeline: TC text -> parse -> semantic analysis + range inference ->
// input checks -> backend mapper -> executor.  Counterpart of tc/core/compiler.h:71-98,
// compiler-inl.h:34-76 and compiler.cc:56-124.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "tc/core/ir.h"
#include "tc/core/tensor.h"
#include "tc/lang/tree.h"
#include "tc/utils/compiler_options.h"

namespace tc {
namespace detail {

// Every def in the TC string, keyed by name.
std::map<std::string, lang::TreeRef> parse(const std::string& tc);

// Arity, element type, rank and stride sanity of the inputs against the definition; throws
// lang::ErrorReport or InvalidStrideException.
void checkInputsCompliant(const ir::Function& f, const std::vector<const DLConstTensor*>& inputs);

ir::Function translate(
    const lang::TreeRef& def, const std::vector<const DLConstTensor*>& inputs, const CompilerOptions& options);

std::vector<TensorInfo> inferOutputTensorInfo(
    const lang::TreeRef& def, const std::vector<const DLConstTensor*>& inputs, const CompilerOptions& options);

// The executor of a mapped function: JIT-compiles `result` (the second half of compile(), for
// callers that look at the mapper's output before they decide to compile it).
template <typename Backend>
std::unique_ptr<typename Backend::ExecutorType> makeExecutor(
    const ir::Function& f,
    const std::vector<const DLConstTensor*>& inputs,
    const typename Backend::CompilationResultType& result) {
  std::vector<TensorInfo> inputsInfo = makeTensorInfoVector(inputs);
  std::vector<TensorInfo> outputsInfo;
  for (const auto& o : f.outputs) {
    outputsInfo.emplace_back(o.type.toDL(), 0, o.extents, makeStridesFromSizes(o.extents));
  }
  return std::unique_ptr<typename Backend::ExecutorType>(
      new typename Backend::ExecutorType(inputsInfo, outputsInfo, f, result));
}

template <typename Backend>
std::unique_ptr<typename Backend::ExecutorType> compile(
    const lang::TreeRef& def,
    const std::vector<const DLConstTensor*>& inputs,
    const typename Backend::MappingOptionsType& options,
    const CompilerOptions& compilerOptions = CompilerOptions()) {
  ir::Function f = translate(def, inputs, compilerOptions);
  checkInputsCompliant(f, inputs);
  return makeExecutor<Backend>(f, inputs, Backend::compileWithTcMapper(f.name, f, inputs, options));
}

} // namespace detail

// Shapes, element types and contiguous strides of the outputs `entryPoint` produces for these inputs.
std::vector<TensorInfo> inferOutputTensorInfo(
    const std::string& tc,
    const std::string& entryPoint,
    const std::vector<const DLConstTensor*>& inputs,
    const CompilerOptions& compilerOptions = CompilerOptions());

template <typename Backend>
std::unique_ptr<typename Backend::ExecutorType> compile(
    const std::string& tc,
    const std::string& entryPoint,
    const std::vector<const DLConstTensor*>& inputs,
    const typename Backend::MappingOptionsType& options,
    const CompilerOptions& compilerOptions = CompilerOptions()) {
  auto defs = detail::parse(tc);
  auto it = defs.find(entryPoint);
  if (it == defs.end()) {
    throw std::runtime_error("attempting to access undefined function " + entryPoint);
  }
  return detail::compile<Backend>(it->second, inputs, options, compilerOptions);
}

} // namespace tc
