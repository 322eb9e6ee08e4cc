#include "tc/core/hip/hip.h"

namespace tc {

HipGPUInfo::HipGPUInfo() {
  int n = 0;
  if (tchip_device_count(&n) != 0) {
    n = 0;
  }
  for (int i = 0; i < n; ++i) {
    char name[256] = {0}, arch[64] = {0};
    size_t lds = 65536;
    if (tchip_device_name(i, name, sizeof(name)) != 0 || tchip_device_arch(i, arch, sizeof(arch)) != 0) {
      break;
    }
    tchip_device_lds_bytes(i, &lds);
    names_.push_back(name);
    archs_.push_back(arch);
    lds_.push_back(lds);
  }
}

HipGPUInfo& HipGPUInfo::GPUInfo() {
  static thread_local HipGPUInfo info;
  return info;
}

int HipGPUInfo::CurrentGPUId() const {
  int d = 0;
  if (names_.empty() || tchip_get_device(&d) != 0) {
    return 0;
  }
  return d;
}
std::string HipGPUInfo::GetGPUName(int id) const {
  if (names_.empty()) return "";
  return names_.at(id < 0 ? CurrentGPUId() : id);
}
std::string HipGPUInfo::GetArch(int id) const {
  if (archs_.empty()) return "gfx950";
  return archs_.at(id < 0 ? CurrentGPUId() : id);
}
size_t HipGPUInfo::SharedMemorySize() const {
  if (lds_.empty()) return 65536;
  return lds_.at(CurrentGPUId());
}

} // namespace tc
