// Implementation of the thin HIP C ABI declared in include/tchip.h.
//
// The HIP runtime and hipRTC are bound at run time, not at link time: a process must talk to one
// HIP runtime only (streams, events and modules are objects of the runtime that created them),
// and a host framework such as PyTorch ships and loads its own copy.  The loader therefore
// prefers a runtime that is already mapped into the process and only falls back to the system
// one (ROCm's libamdhip64.so.N / libhiprtc.so.N).
#include "tchip.h"

#include <dlfcn.h>
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace {
thread_local std::string g_lastError;

struct HipApi {
  void* hipLib = nullptr;
  void* rtcLib = nullptr;
  std::string loadError;
#define TCHIP_FN(name) decltype(&::name) name = nullptr
  TCHIP_FN(hipGetDeviceCount);
  TCHIP_FN(hipGetDevice);
  TCHIP_FN(hipSetDevice);
  hipError_t (*hipGetDevicePropertiesFn)(hipDeviceProp_t*, int) = nullptr;
  TCHIP_FN(hipDeviceSynchronize);
  TCHIP_FN(hipStreamSynchronize);
  TCHIP_FN(hipModuleLoadData);
  TCHIP_FN(hipModuleGetFunction);
  TCHIP_FN(hipModuleUnload);
  TCHIP_FN(hipModuleLaunchKernel);
  TCHIP_FN(hipEventCreate);
  TCHIP_FN(hipEventRecord);
  TCHIP_FN(hipEventSynchronize);
  TCHIP_FN(hipEventElapsedTime);
  TCHIP_FN(hipEventDestroy);
  TCHIP_FN(hipGetLastError);
  TCHIP_FN(hipGetErrorString);
  hipError_t (*hipMallocFn)(void**, size_t) = nullptr;
  TCHIP_FN(hipFree);
  TCHIP_FN(hipMemcpy);
  TCHIP_FN(hiprtcCreateProgram);
  TCHIP_FN(hiprtcCompileProgram);
  TCHIP_FN(hiprtcGetProgramLogSize);
  TCHIP_FN(hiprtcGetProgramLog);
  TCHIP_FN(hiprtcGetCodeSize);
  TCHIP_FN(hiprtcGetCode);
  TCHIP_FN(hiprtcDestroyProgram);
  TCHIP_FN(hiprtcGetErrorString);
#undef TCHIP_FN

  static void* openFirst(const std::vector<const char*>& names) {
    for (const char* n : names) { // a copy the process already uses wins
      if (void* h = dlopen(n, RTLD_NOW | RTLD_GLOBAL | RTLD_NOLOAD)) return h;
    }
    for (const char* n : names) {
      if (void* h = dlopen(n, RTLD_NOW | RTLD_GLOBAL)) return h;
    }
    return nullptr;
  }
  template <typename F>
  bool bind(void* lib, const char* sym, F& out) {
    out = reinterpret_cast<F>(dlsym(lib, sym));
    if (!out) loadError += std::string(loadError.empty() ? "missing symbols: " : ", ") + sym;
    return out != nullptr;
  }
  HipApi() {
    hipLib = openFirst({"libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6", "/opt/rocm/lib/libamdhip64.so"});
    // hipRTC is a stand-alone compiler (it shares no state with the runtime): TCHIP_HIPRTC names a
    // specific copy, e.g. a newer ROCm's next to the runtime an older framework build brought along
    if (const char* forced = std::getenv("TCHIP_HIPRTC")) {
      rtcLib = dlopen(forced, RTLD_NOW | RTLD_LOCAL);
      if (!rtcLib) loadError = std::string("cannot load TCHIP_HIPRTC=") + forced + ": " + dlerror();
    } else {
      rtcLib = openFirst({"libhiprtc.so", "libhiprtc.so.7", "libhiprtc.so.6", "/opt/rocm/lib/libhiprtc.so"});
    }
    if (!hipLib) loadError = "cannot load the HIP runtime (libamdhip64.so)";
    if (!rtcLib && loadError.find("TCHIP_HIPRTC") == std::string::npos) {
      loadError += std::string(loadError.empty() ? "" : "; ") + "cannot load hipRTC (libhiprtc.so)";
    }
    if (hipLib) {
#define TCHIP_BIND(name) bind(hipLib, #name, name)
      TCHIP_BIND(hipGetDeviceCount);
      TCHIP_BIND(hipGetDevice);
      TCHIP_BIND(hipSetDevice);
      bind(hipLib, "hipGetDevicePropertiesR0600", hipGetDevicePropertiesFn);
      TCHIP_BIND(hipDeviceSynchronize);
      TCHIP_BIND(hipStreamSynchronize);
      TCHIP_BIND(hipModuleLoadData);
      TCHIP_BIND(hipModuleGetFunction);
      TCHIP_BIND(hipModuleUnload);
      TCHIP_BIND(hipModuleLaunchKernel);
      TCHIP_BIND(hipEventCreate);
      TCHIP_BIND(hipEventRecord);
      TCHIP_BIND(hipEventSynchronize);
      TCHIP_BIND(hipEventElapsedTime);
      TCHIP_BIND(hipEventDestroy);
      TCHIP_BIND(hipGetLastError);
      TCHIP_BIND(hipGetErrorString);
      bind(hipLib, "hipMalloc", hipMallocFn);
      TCHIP_BIND(hipFree);
      TCHIP_BIND(hipMemcpy);
#undef TCHIP_BIND
    }
    if (rtcLib) {
#define TCHIP_BIND(name) bind(rtcLib, #name, name)
      TCHIP_BIND(hiprtcCreateProgram);
      TCHIP_BIND(hiprtcCompileProgram);
      TCHIP_BIND(hiprtcGetProgramLogSize);
      TCHIP_BIND(hiprtcGetProgramLog);
      TCHIP_BIND(hiprtcGetCodeSize);
      TCHIP_BIND(hiprtcGetCode);
      TCHIP_BIND(hiprtcDestroyProgram);
      TCHIP_BIND(hiprtcGetErrorString);
#undef TCHIP_BIND
    }
  }
};

HipApi& api() {
  static HipApi a;
  return a;
}

constexpr int kNotLoaded = 20000;
bool hipReady() {
  if (api().loadError.empty()) return true;
  g_lastError = api().loadError;
  return false;
}

int fail(hipError_t e, const char* what) {
  g_lastError = std::string(what) + ": " + api().hipGetErrorString(e);
  return static_cast<int>(e);
}
int failRtc(hiprtcResult r, const char* what) {
  g_lastError = std::string(what) + ": " + api().hiprtcGetErrorString(r);
  return 10000 + static_cast<int>(r);
}
#define TCHIP_TRY(call)                   \
  do {                                    \
    if (!hipReady()) return kNotLoaded;   \
    hipError_t e_ = (api().call);         \
    if (e_ != hipSuccess) {               \
      return fail(e_, #call);             \
    }                                     \
  } while (0)

char* dupString(const std::string& s) {
  char* p = static_cast<char*>(std::malloc(s.size() + 1));
  if (p) {
    std::memcpy(p, s.c_str(), s.size() + 1);
  }
  return p;
}

// device properties through the versioned entry point; a generously sized buffer guards against
// a runtime whose struct is larger than this build's header
int deviceProps(int device, hipDeviceProp_t* out) {
  if (!hipReady()) return kNotLoaded;
  std::vector<char> buf(sizeof(hipDeviceProp_t) + 4096, 0);
  hipError_t e = api().hipGetDevicePropertiesFn(reinterpret_cast<hipDeviceProp_t*>(buf.data()), device);
  if (e != hipSuccess) return fail(e, "hipGetDeviceProperties");
  std::memcpy(out, buf.data(), sizeof(hipDeviceProp_t));
  return 0;
}
} // namespace

extern "C" {

int tchip_device_count(int* count) {
  TCHIP_TRY(hipGetDeviceCount(count));
  return 0;
}
int tchip_get_device(int* device) {
  TCHIP_TRY(hipGetDevice(device));
  return 0;
}
int tchip_set_device(int device) {
  TCHIP_TRY(hipSetDevice(device));
  return 0;
}
int tchip_malloc(void** ptr, size_t bytes) {
  TCHIP_TRY(hipMallocFn(ptr, bytes));
  return 0;
}
int tchip_free_device(void* ptr) {
  TCHIP_TRY(hipFree(ptr));
  return 0;
}
int tchip_memcpy_to_device(void* dst, const void* src, size_t bytes) {
  TCHIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return 0;
}
int tchip_memcpy_to_host(void* dst, const void* src, size_t bytes) {
  TCHIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return 0;
}
int tchip_device_name(int device, char* buf, size_t n) {
  hipDeviceProp_t p;
  if (int st = deviceProps(device, &p)) return st;
  // (the marketing name comes from a table that an installation may lack: the architecture
  // string then identifies the device)
  std::strncpy(buf, p.name[0] ? p.name : p.gcnArchName, n);
  if (n) buf[n - 1] = '\0';
  return 0;
}
int tchip_device_arch(int device, char* buf, size_t n) {
  hipDeviceProp_t p;
  if (int st = deviceProps(device, &p)) return st;
  std::string arch = p.gcnArchName; // "gfx950:sramecc+:xnack-"
  arch = arch.substr(0, arch.find(':'));
  std::strncpy(buf, arch.c_str(), n);
  if (n) buf[n - 1] = '\0';
  return 0;
}
int tchip_device_lds_bytes(int device, size_t* bytes) {
  hipDeviceProp_t p;
  if (int st = deviceProps(device, &p)) return st;
  *bytes = p.sharedMemPerBlock;
  return 0;
}
int tchip_device_compute_units(int device, int* count) {
  hipDeviceProp_t p;
  if (int st = deviceProps(device, &p)) return st;
  *count = p.multiProcessorCount;
  return 0;
}
int tchip_sync_device(void) {
  TCHIP_TRY(hipDeviceSynchronize());
  return 0;
}
int tchip_stream_sync(tchip_stream_t stream) {
  TCHIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}

int tchip_rtc_compile(
    const char* source, const char* name, const char* arch,
    const char* const* flags, int numFlags, char** code, size_t* codeSize, char** log) {
  *code = nullptr;
  *codeSize = 0;
  if (log) *log = nullptr;
  if (!hipReady()) return kNotLoaded;
  hiprtcProgram prog;
  hiprtcResult r = api().hiprtcCreateProgram(&prog, source, name, 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) {
    return failRtc(r, "hiprtcCreateProgram");
  }
  std::string archFlag = std::string("--offload-arch=") + arch;
  std::vector<const char*> opts{archFlag.c_str()};
  for (int i = 0; i < numFlags; ++i) {
    opts.push_back(flags[i]);
  }
  r = api().hiprtcCompileProgram(prog, static_cast<int>(opts.size()), opts.data());
  size_t logSize = 0;
  api().hiprtcGetProgramLogSize(prog, &logSize);
  std::string logText(logSize, '\0');
  if (logSize) {
    api().hiprtcGetProgramLog(prog, &logText[0]);
  }
  if (log) *log = dupString(logText);
  if (r != HIPRTC_SUCCESS) {
    api().hiprtcDestroyProgram(&prog);
    g_lastError = std::string("hiprtcCompileProgram: ") + api().hiprtcGetErrorString(r) + "\n" + logText;
    return 10000 + static_cast<int>(r);
  }
  size_t n = 0;
  r = api().hiprtcGetCodeSize(prog, &n);
  if (r == HIPRTC_SUCCESS) {
    *code = static_cast<char*>(std::malloc(n));
    r = *code ? api().hiprtcGetCode(prog, *code) : HIPRTC_ERROR_OUT_OF_MEMORY;
  }
  api().hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    std::free(*code);
    *code = nullptr;
    return failRtc(r, "hiprtcGetCode");
  }
  *codeSize = n;
  return 0;
}
void tchip_free(void* p) {
  std::free(p);
}

int tchip_module_load(const void* code, tchip_module_t* module) {
  hipModule_t m;
  TCHIP_TRY(hipModuleLoadData(&m, code));
  *module = m;
  return 0;
}
int tchip_module_get_function(tchip_module_t module, const char* name, tchip_function_t* fn) {
  hipFunction_t f;
  TCHIP_TRY(hipModuleGetFunction(&f, static_cast<hipModule_t>(module), name));
  *fn = f;
  return 0;
}
int tchip_module_unload(tchip_module_t module) {
  TCHIP_TRY(hipModuleUnload(static_cast<hipModule_t>(module)));
  return 0;
}

int tchip_launch(
    tchip_function_t fn, const unsigned grid[3], const unsigned block[3],
    unsigned dynamicLds, tchip_stream_t stream, void** args) {
  TCHIP_TRY(hipModuleLaunchKernel(
      static_cast<hipFunction_t>(fn), grid[0], grid[1], grid[2], block[0], block[1], block[2],
      dynamicLds, static_cast<hipStream_t>(stream), args, nullptr));
  return 0;
}

int tchip_event_create(tchip_event_t* ev) {
  hipEvent_t e;
  TCHIP_TRY(hipEventCreate(&e));
  *ev = e;
  return 0;
}
int tchip_event_record(tchip_event_t ev, tchip_stream_t stream) {
  TCHIP_TRY(hipEventRecord(static_cast<hipEvent_t>(ev), static_cast<hipStream_t>(stream)));
  return 0;
}
int tchip_event_sync(tchip_event_t ev) {
  TCHIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(ev)));
  return 0;
}
int tchip_event_elapsed_ms(tchip_event_t start, tchip_event_t stop, float* ms) {
  TCHIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return 0;
}
int tchip_event_destroy(tchip_event_t ev) {
  TCHIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(ev)));
  return 0;
}
int tchip_get_last_error(void) {
  if (!hipReady()) return kNotLoaded;
  hipError_t e = api().hipGetLastError();
  if (e != hipSuccess) {
    fail(e, "hipGetLastError");
  }
  return static_cast<int>(e);
}
const char* tchip_last_error_string(void) {
  return g_lastError.c_str();
}

} // extern "C"
