#include "tc/core/hip/hip_rtc.h"

#include <array>
#include <iostream>

#include "tc/core/check.h"
#include "tc/core/flags.h"

namespace tc {

namespace {
// A pair of timing events that is destroyed on every way out of a launch, an exception thrown
// by a failed driver call included (the tuner catches those and carries on with the next
// candidate, so a leak per failed candidate would add up over a tuning run).
struct EventPair {
  tchip_event_t start = nullptr, stop = nullptr;
  void create() {
    TC_HIP_CHECK(tchip_event_create(&start));
    TC_HIP_CHECK(tchip_event_create(&stop));
  }
  ~EventPair() {
    if (start) tchip_event_destroy(start);
    if (stop) tchip_event_destroy(stop);
  }
};
} // namespace

HipRTCFunction::~HipRTCFunction() {
  if (!cleared_) {
    try {
      clear();
    } catch (...) {
    }
  }
}

void HipRTCFunction::clear() {
  std::unique_lock<std::shared_mutex> lock(mutex_);
  if (cleared_) return;
  for (auto& m : modules_) {
    int old = 0;
    if (tchip_get_device(&old) == 0) {
      tchip_set_device(m.first);
      tchip_module_unload(m.second);
      tchip_set_device(old);
    }
  }
  modules_.clear();
  functions_.clear();
  cleared_ = true;
}

std::unique_ptr<HipRTCFunction> HipRTCFunction::Compile(const std::string& name, const std::string& source) {
  std::unique_ptr<HipRTCFunction> res(new HipRTCFunction());
  res->name_ = name;
  std::string arch = HipGPUInfo::GPUInfo().GetArch();
  // Packed-FP32 instruction selection is switched off for all device code of this library.
  // Kernel arguments (the size parameters and the tensor pointers) arrive in scalar registers
  // with the wavefront instead of being fetched by its first instructions: the group convolution
  // of 10 us starts 0.1 us earlier in every wavefront (-amdgpu-kernarg-preload-count, at most 16
  // dwords; arguments beyond that are loaded as before).
  std::vector<const char*> opts = {"-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                                   "-mllvm", "-amdgpu-kernarg-preload-count=16"};
  // (-munsafe-fp-atomics, only for programs with a reduction divided among blocks: floating-point
  // atomic adds become the hardware instruction, which is exact for tensors in ordinary,
  // coarse-grained device memory and may lose updates in fine-grained or managed allocations)
  if (source.find("__tc::atomicAccumulate(&") != std::string::npos || source.find("__tc::atomicCombine<") != std::string::npos) {
    opts.push_back("-munsafe-fp-atomics");
  }
  if (tc::flags().fast_math) opts.push_back("-ffast-math");
  char* code = nullptr;
  char* log = nullptr;
  size_t size = 0;
  int status = tchip_rtc_compile(
      source.c_str(), (name + ".hip").c_str(), arch.c_str(), opts.data(), static_cast<int>(opts.size()), &code, &size, &log);
  std::string logText = log ? log : "";
  tchip_free(log);
  if (status != 0) {
    tchip_free(code);
    throw std::runtime_error("hipRTC compilation of " + name + " failed:\n" + logText + "\n--- source ---\n" + source);
  }
  res->code_.assign(code, size);
  tchip_free(code);
  return res;
}

Duration HipRTCFunction::Launch(
    const std::vector<HipKernelLaunch>& kernels,
    tchip_stream_t stream,
    std::vector<int> params,
    std::vector<void*> outputs,
    std::vector<const void*> inputs,
    bool profile,
    int repeats) const {
  int dev = 0;
  TC_HIP_CHECK(tchip_get_device(&dev));
  std::vector<tchip_function_t> fns;
  // every handle of this launch, if all of them are there (call with the lock held)
  auto lookUp = [&]() {
    fns.clear();
    if (!modules_.count(dev)) return false;
    for (const auto& k : kernels) {
      auto it = functions_.find(std::make_pair(dev, k.name));
      if (it == functions_.end()) return false;
      fns.push_back(it->second);
    }
    return true;
  };
  std::shared_lock<std::shared_mutex> launching(mutex_);
  TC_CHECK(!cleared_) << "launch of a cleared RTC function";
  if (!lookUp()) {
    // the per-device module and function handles are filled in lazily: one thread at a time
    launching.unlock();
    {
      std::unique_lock<std::shared_mutex> loading(mutex_);
      TC_CHECK(!cleared_) << "launch of a cleared RTC function";
      if (!modules_.count(dev)) {
        tchip_module_t m = nullptr;
        TC_HIP_CHECK(tchip_module_load(code_.data(), &m));
        modules_[dev] = m;
      }
      for (const auto& k : kernels) {
        auto key = std::make_pair(dev, k.name);
        if (!functions_.count(key)) {
          tchip_function_t fn = nullptr;
          TC_HIP_CHECK(tchip_module_get_function(modules_[dev], k.name.c_str(), &fn));
          functions_.emplace(key, fn);
        }
      }
    }
    launching.lock();
    // (a clear() may have run in between: then the launch is refused, never made on stale handles)
    TC_CHECK(!cleared_ && lookUp()) << "launch of a cleared RTC function";
  }
  std::vector<void*> args;
  for (auto& p : params) args.push_back(&p);
  for (auto& p : outputs) args.push_back(&p);
  for (auto& p : inputs) args.push_back((void*)&p);
  TC_CHECK_LE(args.size(), 100u) << "too many kernel arguments";
  EventPair ev;
  if (profile) {
    ev.create();
    TC_HIP_CHECK(tchip_event_record(ev.start, stream));
  }
  for (int r = 0; r < repeats; ++r) {
    for (size_t i = 0; i < kernels.size(); ++i) {
      TC_HIP_CHECK(tchip_launch(fns[i], kernels[i].grid.data(), kernels[i].block.data(), 0, stream, args.data()));
    }
  }
  if (profile) {
    float ms = 0;
    TC_HIP_CHECK(tchip_event_record(ev.stop, stream));
    TC_HIP_CHECK(tchip_event_sync(ev.stop));
    TC_HIP_CHECK(tchip_event_elapsed_ms(ev.start, ev.stop, &ms));
    return Duration::fromNanoSeconds(static_cast<int64_t>(static_cast<double>(ms) * 1e6 + 0.5));
  }
  return Duration::max();
}

} // namespace tc
