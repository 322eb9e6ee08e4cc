// Host-side view of the HIP device: error checking over the tchip C ABI, device information
// and the RAII device guard.  Counterpart of tc/core/cuda/cuda.h:38-131 and cuda.cc:33-104.
#pragma once
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "tchip.h"

#define TC_HIP_CHECK(call)                                                                     \
  do {                                                                                         \
    int status_ = (call);                                                                      \
    if (status_ != 0) {                                                                        \
      std::stringstream ss_;                                                                   \
      ss_ << "HIP error " << status_ << " in " #call " at " << __FILE__ << ":" << __LINE__    \
          << ": " << tchip_last_error_string();                                                \
      throw std::runtime_error(ss_.str());                                                     \
    }                                                                                          \
  } while (0)

namespace tc {

// Names, architectures and LDS sizes of the visible devices, queried once per thread.
class HipGPUInfo {
 public:
  static HipGPUInfo& GPUInfo();
  int NumberGPUs() const { return static_cast<int>(names_.size()); }
  int CurrentGPUId() const;
  std::string GetGPUName(int id = -1) const;  // "" when no device is present
  std::string GetArch(int id = -1) const;     // "gfx950" when no device is present
  size_t SharedMemorySize() const;            // LDS per workgroup; 65536 when no device is present

 private:
  HipGPUInfo();
  std::vector<std::string> names_, archs_;
  std::vector<size_t> lds_;
};

struct WithHipDevice {
  explicit WithHipDevice(size_t g) : newDevice(static_cast<int>(g)) {
    TC_HIP_CHECK(tchip_get_device(&oldDevice));
    TC_HIP_CHECK(tchip_set_device(newDevice));
  }
  ~WithHipDevice() noexcept(false) { TC_HIP_CHECK(tchip_set_device(oldDevice)); }
  int oldDevice = 0;
  int newDevice;
};

} // namespace tc
