/* tchip — the thin C ABI between the TC host library and the HIP runtime / hipRTC.
 *
 * Every HIP entry point the backend needs goes through one of these functions; they replace
 * the CUDA driver / NVRTC call sites of the reference backend, cited per function
 * (paths relative to the reference checkout).  All functions return 0 on success or a non-zero
 * HIP / hipRTC status; no C++ exception crosses this boundary.  tchip_last_error_string()
 * describes the most recent failure on the calling thread.
 */
#ifndef TCHIP_H
#define TCHIP_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef void* tchip_module_t;
typedef void* tchip_function_t;
typedef void* tchip_event_t;
typedef void* tchip_stream_t; /* a hipStream_t; NULL is the default stream */

/* device queries — cudaGetDeviceCount / GetDeviceProperties / Get,SetDevice
 * (tc/core/cuda/cuda.cc:33-55, tc/core/cuda/cuda.h:79-91) */
int tchip_device_count(int* count);
int tchip_get_device(int* device);
int tchip_set_device(int device);
int tchip_device_name(int device, char* buf, size_t buf_size);
int tchip_device_arch(int device, char* buf, size_t buf_size); /* e.g. "gfx950" */
int tchip_device_lds_bytes(int device, size_t* bytes);         /* LDS usable by one workgroup */
int tchip_device_compute_units(int device, int* count);
int tchip_sync_device(void);                                   /* cuda.cc:88-90 */
int tchip_stream_sync(tchip_stream_t stream);

/* device memory for callers that hold no tensor library of their own (the reference leaves
 * allocation to ATen, tc/aten/aten_compiler.cc:46-67): hipMalloc / hipFree and synchronous copies */
int tchip_malloc(void** ptr, size_t bytes);
int tchip_free_device(void* ptr);
int tchip_memcpy_to_device(void* dst, const void* src, size_t bytes);
int tchip_memcpy_to_host(void* dst, const void* src, size_t bytes);

/* JIT — nvrtcCreateProgram / CompileProgram / GetProgramLog / GetPTX
 * (tc/core/cuda/cuda_rtc.cc:208-262).  `arch` like "gfx950"; `flags` are extra compiler
 * options.  On return *code / *log are malloc'ed (free with tchip_free); *log is set even
 * when compilation fails. */
int tchip_rtc_compile(
    const char* source, const char* name, const char* arch,
    const char* const* flags, int num_flags,
    char** code, size_t* code_size, char** log);
void tchip_free(void* p);

/* modules — cuModuleLoadData / GetFunction / Unload (cuda_rtc.cc:45-53,310-329) */
int tchip_module_load(const void* code, tchip_module_t* module);
int tchip_module_get_function(tchip_module_t module, const char* name, tchip_function_t* fn);
int tchip_module_unload(tchip_module_t module);

/* launch — cuLaunchKernel (cuda_rtc.cc:331-366).  `args` holds one pointer per kernel argument. */
int tchip_launch(
    tchip_function_t fn, const unsigned grid[3], const unsigned block[3],
    unsigned dynamic_lds_bytes, tchip_stream_t stream, void** args);

/* events — cudaEventCreate / Record / Synchronize / ElapsedTime / Destroy (cuda_rtc.cc:373-386) */
int tchip_event_create(tchip_event_t* ev);
int tchip_event_record(tchip_event_t ev, tchip_stream_t stream);
int tchip_event_sync(tchip_event_t ev);
int tchip_event_elapsed_ms(tchip_event_t start, tchip_event_t stop, float* ms);
int tchip_event_destroy(tchip_event_t ev);

/* drains and returns the sticky error state — cudaGetLastError
 * (tc/autotuner/cuda/autotuner.cc:134-154) */
int tchip_get_last_error(void);
const char* tchip_last_error_string(void);

#ifdef __cplusplus
}
#endif
#endif /* TCHIP_H */
