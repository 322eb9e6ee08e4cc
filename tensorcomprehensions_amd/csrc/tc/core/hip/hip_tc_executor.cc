#include "tc/core/hip/hip_tc_executor.h"

#include <iostream>

#include "tc/core/flags.h"

namespace tc {

namespace {
// kernel name = TC name + "_" + every size value (tc/core/cuda/cuda_tc_executor.cc:33-43)
std::string specializedKernelName(const std::string& tcName, const ir::Function& f) {
  std::string n = tcName;
  for (const auto& p : f.params) {
    n += "_" + std::to_string(p.second);
  }
  return n;
}
} // namespace

namespace {
template <typename DLT>
void checkPlacement(const std::vector<const DLT*>& ts, const char* what, int currentDevice) {
  for (size_t i = 0; i < ts.size(); ++i) {
    const DLT* t = ts[i];
    if (currentDevice < 0) {
      TC_CHECK(t->ctx.device_type == kDLROCM)
          << what << " " << i << " is not in HIP device memory (DLPack device type " << static_cast<int>(t->ctx.device_type)
          << ", expected " << static_cast<int>(kDLROCM) << "): kernels cannot be launched on it";
      bool empty = false;
      for (int d = 0; d < t->ndim; ++d) empty |= t->shape[d] == 0;
      TC_CHECK(t->data != nullptr || empty) << what << " " << i << " has a null data pointer";
    } else {
      TC_CHECK_EQ(t->ctx.device_id, currentDevice)
          << what << " " << i << " lives on device " << t->ctx.device_id << " but the current device is " << currentDevice;
    }
  }
}
} // namespace

void HipBackend::checkTensorsAreLaunchable(
    const std::vector<const DLConstTensor*>& inputs, const std::vector<const DLTensor*>& outputs, int dev) {
  checkPlacement(inputs, "input", -1);
  checkPlacement(outputs, "output", -1);
  if (dev < 0) TC_HIP_CHECK(tchip_get_device(&dev));
  checkPlacement(inputs, "input", dev);
  checkPlacement(outputs, "output", dev);
}

HipCompilationResult HipBackend::compileWithTcMapper(
    const std::string& tcName,
    const ir::Function& function,
    const std::vector<const DLConstTensor*>& /*inputs*/,
    const HipMappingOptions& options) {
  mapper::DeviceLimits limits;
  limits.ldsBytesPerBlock = static_cast<int64_t>(HipGPUInfo::GPUInfo().SharedMemorySize());
  HipCompilationResult r;
  r.specializedName = specializedKernelName(tcName, function);
  r.program = mapper::mapToHip(function, options, r.specializedName, limits);
  r.source = r.program.source;
  for (auto v : r.program.paramValues) {
    r.parameters.push_back(static_cast<int>(v));
  }
  for (const auto& k : r.program.kernels) {
    HipKernelLaunch l;
    l.name = k.name;
    for (int a = 0; a < 3; ++a) {
      l.grid[a] = static_cast<unsigned>(k.grid[a]);
      l.block[a] = static_cast<unsigned>(k.block[a]);
    }
    r.kernels.push_back(l);
  }
  const auto& k0 = r.program.kernels.front();
  r.grid = HipGrid(std::vector<uint64_t>{(uint64_t)k0.grid[0], (uint64_t)k0.grid[1], (uint64_t)k0.grid[2]});
  r.block = HipBlock(std::vector<uint64_t>{(uint64_t)k0.block[0], (uint64_t)k0.block[1], (uint64_t)k0.block[2]});
  if (flags().debug_tc_mapper) {
    // (the reference logs the options and its schedule trees here, cuda_tc_executor.cc:65-105)
    std::cerr << "[MAPPER] " << r.specializedName << " under " << options.toText() << "\n";
    for (const auto& k : r.kernels) {
      std::cerr << "[MAPPER]   kernel " << k.name << " grid " << k.grid[0] << "x" << k.grid[1] << "x" << k.grid[2] << " block "
                << k.block[0] << "x" << k.block[1] << "x" << k.block[2] << "\n";
    }
  }
  if (flags().dump_hip) {
    std::cerr << "generated HIP for " << r.specializedName << ":\n" << r.source << std::endl;
  }
  return r;
}

HipTcExecutor::HipTcExecutor(
    const std::vector<TensorInfo>& inputsInfo,
    const std::vector<TensorInfo>& outputsInfo,
    const ir::Function& function,
    const HipCompilationResult& compilationResult)
    : TcExecutor<HipBackend>(inputsInfo, outputsInfo, function, compilationResult),
      result_(compilationResult) {
  // the JIT runs here, on the calling thread; nothing touches the device until the first launch
  rtcFun_ = HipRTCFunction::Compile(result_.specializedName, result_.source);
}

void HipTcExecutor::uncheckedRun(
    const std::vector<const void*>& inputs,
    const std::vector<void*>& outputs,
    HipRuntimeInformation info) const {
  TC_CHECK(rtcFun_) << "No rtcFun_ attached, cannot launch";
  rtcFun_->Launch(result_.kernels, info.stream, result_.parameters, outputs, inputs, false);
}

Duration HipTcExecutor::profileRepeated(
    const std::vector<const void*>& inputs,
    const std::vector<void*>& outputs,
    int repeats,
    HipRuntimeInformation info) const {
  TC_CHECK(rtcFun_) << "No rtcFun_ attached, cannot launch";
  TC_CHECK_GE(repeats, 1);
  return rtcFun_->Launch(result_.kernels, info.stream, result_.parameters, outputs, inputs, true, repeats);
}

ProfilingInfo HipTcExecutor::profileUnchecked(
    const std::vector<const void*>& inputs,
    const std::vector<void*>& outputs,
    HipRuntimeInformation info) const {
  TC_CHECK(rtcFun_) << "No rtcFun_ attached, cannot launch";
  auto t0 = std::chrono::steady_clock::now();
  Duration kernel = rtcFun_->Launch(result_.kernels, info.stream, result_.parameters, outputs, inputs, true);
  Duration wall = Duration::since(t0);
  return ProfilingInfo{wall > kernel ? wall - kernel : Duration::zero(), kernel};
}

} // namespace tc
