// JIT-compiled HIP module: compile with hipRTC, load lazily per device, launch, time.
// Four verbs as in the reference's CudaRTCFunction (tc/core/cuda/cuda_rtc.h:38-70,
// cuda_rtc.cc:265-387): Compile, Launch, clear, destructor.  One module may hold several
// kernels (a TC that maps to more than one launch).
#pragma once
#include <array>
#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <vector>

#include "tc/core/hip/hip.h"
#include "tc/core/utils/time.h"

namespace tc {

struct HipKernelLaunch {
  std::string name;
  std::array<unsigned, 3> grid, block;
};

class HipRTCFunction {
 public:
  ~HipRTCFunction();
  // Throws std::runtime_error carrying the compiler log when compilation fails.
  static std::unique_ptr<HipRTCFunction> Compile(const std::string& name, const std::string& source);

  // Launches the kernels in order on `stream` with arguments (params..., outputs..., inputs...).
  // With profile=true the launches are bracketed by events and the elapsed device time is
  // returned after synchronising; otherwise returns Duration::max() without synchronising.
  // `repeats` > 1 issues the whole launch sequence that many times back to back (between the
  // events when profiling): the way to time kernels shorter than a launch round trip.
  Duration Launch(
      const std::vector<HipKernelLaunch>& kernels,
      tchip_stream_t stream,
      std::vector<int> params,
      std::vector<void*> outputs,
      std::vector<const void*> inputs,
      bool profile = false,
      int repeats = 1) const;

  void clear();
  const std::string& code() const { return code_; }

 private:
  HipRTCFunction() = default;
  std::string name_;
  std::string code_; // code object
  // guards the two maps: launches hold it shared from the lookup of their handles to the end of
  // their launch calls, clear() and the lazy loading hold it exclusively, so a module is never
  // unloaded between a lookup and the launch that uses it
  mutable std::shared_mutex mutex_;
  mutable std::map<int, tchip_module_t> modules_;                              // per device id
  mutable std::map<std::pair<int, std::string>, tchip_function_t> functions_;  // (device, kernel)
  bool cleared_ = false;
};

} // namespace tc
