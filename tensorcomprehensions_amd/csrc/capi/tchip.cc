// Implementation of the thin HIP C ABI declared in include/tchip.h.
#include "tchip.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {
thread_local std::string g_lastError;

int fail(hipError_t e, const char* what) {
  g_lastError = std::string(what) + ": " + hipGetErrorString(e);
  return static_cast<int>(e);
}
int failRtc(hiprtcResult r, const char* what) {
  g_lastError = std::string(what) + ": " + hiprtcGetErrorString(r);
  return 10000 + static_cast<int>(r);
}
#define TCHIP_TRY(call)                 \
  do {                                  \
    hipError_t e_ = (call);             \
    if (e_ != hipSuccess) {             \
      return fail(e_, #call);           \
    }                                   \
  } while (0)

char* dupString(const std::string& s) {
  char* p = static_cast<char*>(std::malloc(s.size() + 1));
  if (p) {
    std::memcpy(p, s.c_str(), s.size() + 1);
  }
  return p;
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
int tchip_device_name(int device, char* buf, size_t n) {
  hipDeviceProp_t p;
  TCHIP_TRY(hipGetDeviceProperties(&p, device));
  std::strncpy(buf, p.name, n);
  if (n) buf[n - 1] = '\0';
  return 0;
}
int tchip_device_arch(int device, char* buf, size_t n) {
  hipDeviceProp_t p;
  TCHIP_TRY(hipGetDeviceProperties(&p, device));
  std::string arch = p.gcnArchName; // "gfx950:sramecc+:xnack-"
  arch = arch.substr(0, arch.find(':'));
  std::strncpy(buf, arch.c_str(), n);
  if (n) buf[n - 1] = '\0';
  return 0;
}
int tchip_device_lds_bytes(int device, size_t* bytes) {
  hipDeviceProp_t p;
  TCHIP_TRY(hipGetDeviceProperties(&p, device));
  *bytes = p.sharedMemPerBlock;
  return 0;
}
int tchip_device_compute_units(int device, int* count) {
  hipDeviceProp_t p;
  TCHIP_TRY(hipGetDeviceProperties(&p, device));
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
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, name, 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) {
    return failRtc(r, "hiprtcCreateProgram");
  }
  std::string archFlag = std::string("--offload-arch=") + arch;
  std::vector<const char*> opts{archFlag.c_str()};
  for (int i = 0; i < numFlags; ++i) {
    opts.push_back(flags[i]);
  }
  r = hiprtcCompileProgram(prog, static_cast<int>(opts.size()), opts.data());
  size_t logSize = 0;
  hiprtcGetProgramLogSize(prog, &logSize);
  std::string logText(logSize, '\0');
  if (logSize) {
    hiprtcGetProgramLog(prog, &logText[0]);
  }
  if (log) *log = dupString(logText);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    g_lastError = std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + logText;
    return 10000 + static_cast<int>(r);
  }
  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r == HIPRTC_SUCCESS) {
    *code = static_cast<char*>(std::malloc(n));
    r = *code ? hiprtcGetCode(prog, *code) : HIPRTC_ERROR_OUT_OF_MEMORY;
  }
  hiprtcDestroyProgram(&prog);
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
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fail(e, "hipGetLastError");
  }
  return static_cast<int>(e);
}
const char* tchip_last_error_string(void) {
  return g_lastError.c_str();
}

} // extern "C"
