// The HIP backend's trait bundle: the types and static hooks the backend-generic compile,
// executor and autotuner templates are parameterised on.  Mirror of the reference's CudaBackend
// (tc/core/cuda/cuda_backend.h:34-87).
#pragma once
#include <string>
#include <vector>

#include "tc/core/hip/hip.h"
#include "tc/core/hip/hip_mapping_options.h"
#include "tc/core/hip/hip_rtc.h"
#include "tc/core/ir.h"
#include "tc/core/mapper/mapper.h"
#include "tc/core/tensor.h"

namespace tc {

// What the mapper hands to the executor.
struct HipCompilationResult {
  std::string source;
  std::string specializedName;
  std::vector<int> parameters;           // size values, sorted by parameter name
  HipGrid grid;                          // of the first kernel
  HipBlock block;
  std::vector<HipKernelLaunch> kernels;  // every launch, in order
  mapper::MappedProgram program;         // mapping decisions, for inspection and tests
};

struct HipRuntimeInformation {
  tchip_stream_t stream = nullptr;       // default stream unless set
};

class HipTcExecutor;

struct HipBackend {
  using ExecutorType = HipTcExecutor;
  using MappingOptionsType = HipMappingOptions;
  using CompilationResultType = HipCompilationResult;
  using RTCFunctionType = HipRTCFunction;
  using WithDevice = WithHipDevice;
  using RuntimeInformation = HipRuntimeInformation;
  using MappingOptionsAsCpp = HipMappingOptionsAsCpp;
  using MappingOptionsCppPrinter = HipMappingOptionsCppPrinter;
  // Cache files are written with a hand-rolled proto2 wire codec: the "proto types" are the
  // serialized messages (tc/proto/compcache.proto:20-62 with the HIP options message as value).
  using OptionsCacheProtoType = std::string;
  using OptionsCacheValueProtoType = std::string;

  // device name; part of the tuning-cache key
  static std::string backendString() { return HipGPUInfo::GPUInfo().GetGPUName(); }
  static std::string makeDeviceFilename(const std::string& fn) { return fn + ".hip"; }

  // Throws unless every tensor holds non-null memory of HIP device `device` (-1: the current
  // device).  The device-type and null tests come first and touch no HIP call, so host tensors
  // are refused on a machine without a GPU as well.
  static void checkTensorsAreLaunchable(
      const std::vector<const DLConstTensor*>& inputs, const std::vector<const DLTensor*>& outputs, int device = -1);

  static CompilationResultType compileWithTcMapper(
      const std::string& tcName,
      const ir::Function& function,
      const std::vector<const DLConstTensor*>& inputs,
      const MappingOptionsType& options);
};

} // namespace tc
