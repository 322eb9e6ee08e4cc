/* tc_hip — C ABI of the Tensor Comprehensions HIP backend (library libtc_hip.so).
 *
 * The reference exposes this path as C++ templates over at::Tensor / DLTensor
 * (tc::aten::compile / prepareOutputs / run / profile / uncheckedRun in tc/aten/aten_compiler.h,
 * tc::compile / tc::inferOutputTensorInfo in tc/core/compiler.h, TcExecutor in
 * tc/core/tc_executor.h, ATenAutotuner in tc/aten/aten_autotuner.h).  Each entry point below
 * is the plain-C form of one of those; a binding in any language needs nothing else.
 *
 * Tensors cross the boundary as DLPack-layout structs (DLTensor / DLConstTensor, the types the
 * reference's core API takes, tc/core/tensor.h:36-50).  Data pointers are device pointers and
 * are only borrowed for the duration of a call.  Mapping options cross as text
 * ("preset;key=value;...", keys named like the reference's fluent setters) or as a serialized
 * options message.  Every function returns 0 on success; on failure tc_last_error() returns the
 * message of the C++ exception that was caught on the calling thread (a lang::ErrorReport text
 * with the highlighted source for TC errors).
 */
#ifndef TC_HIP_H
#define TC_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#ifndef TC_DLPACK_TYPES_DEFINED
#define TC_DLPACK_TYPES_DEFINED
typedef struct { int32_t device_type; int32_t device_id; } tc_dl_context;
/* code: 0 int (8, 16, 32, 64 bits), 1 uint (8 = uint8 or bool, 16, 32, 64), 2 float (16, 32, 64) */
typedef struct { uint8_t code; uint8_t bits; uint16_t lanes; } tc_dl_datatype;
typedef struct {
  void* data;
  tc_dl_context ctx;
  int32_t ndim;
  tc_dl_datatype dtype;
  int64_t* shape;
  int64_t* strides; /* NULL = contiguous */
  uint64_t byte_offset;
} tc_dl_tensor;
#endif

#define TC_MAX_RANK 8
typedef struct {
  tc_dl_datatype dtype;
  int32_t ndim;
  int64_t shape[TC_MAX_RANK];
  int64_t strides[TC_MAX_RANK];
} tc_tensor_info;

typedef struct tc_executor tc_executor_t;

const char* tc_last_error(void);
void tc_free(void* p); /* frees strings returned through char** parameters */

/* tc::CompilerOptions (tc/utils/compiler_options.h:27-37) used by the calling thread's next
 * calls: print warnings to stderr / turn warnings into errors.  Defaults: 1, 0. */
void tc_set_compiler_options(int emit_warnings, int throw_warnings);

/* tc::inferOutputTensorInfo (tc/core/compiler.h:88-92; tc::aten::inferOutputTensorInfo,
 * tc/aten/aten_compiler.h:35-38).  Writes up to `capacity` entries, *count = number of outputs. */
int tc_infer_output_info(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs,
    tc_tensor_info* outputs, int capacity, int* count);

/* tc::compile<HipBackend> (tc/core/compiler.h:71-78; tc::aten::compile, aten_compiler.h:56-62).
 * `options` is option text; see tc_options_* below.  With the option reductionBlocks above 1 the
 * kernels add floating-point partial sums with the hardware atomic (hipRTC gets
 * -munsafe-fp-atomics for such sources only): the outputs must then lie in ordinary
 * coarse-grained device memory (hipMalloc, a torch tensor), not in fine-grained or host-mapped
 * allocations. */
int tc_compile(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const char* options, tc_executor_t** executor);
/* same with a serialized options message (HipMappingOptions::toProtobufSerializedString) */
int tc_compile_serialized_options(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const void* options, size_t options_size, tc_executor_t** executor);

/* TcExecutor::run (tc/core/tc_executor.h:89-92; tc::aten::run, aten_compiler.h:69-73):
 * checks count, rank, dtype and shape, launches on `stream` (a hipStream_t or NULL), does not
 * synchronise. */
int tc_executor_run(
    const tc_executor_t* executor,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const tc_dl_tensor* const* outputs, int num_outputs, void* stream);
/* TcExecutor::uncheckedRun (tc_executor.h:109-112; tc::aten::uncheckedRun, aten_compiler.h:88-92):
 * raw device pointers, no checks. */
int tc_executor_unchecked_run(
    const tc_executor_t* executor,
    const void* const* inputs, int num_inputs, void* const* outputs, int num_outputs, void* stream);
/* TcExecutor::profile (tc_executor.h:94-98; tc::aten::profile, aten_compiler.h:79-83):
 * like run, bracketed by device events; synchronises.  Times in microseconds (fractional). */
int tc_executor_profile(
    const tc_executor_t* executor,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const tc_dl_tensor* const* outputs, int num_outputs, void* stream,
    double* kernel_us, double* cpu_overhead_us);

/* `repeats` back-to-back launches between one pair of events on `stream`, raw pointers, no
 * checks; *total_us = device time of all of them.  For kernels shorter than a host launch round
 * trip; the reference's benchmark loop (tc/benchmarks/benchmark_fixture.h:201-241) times single
 * launches at whole-microsecond resolution instead. */
int tc_executor_profile_repeated(
    const tc_executor_t* executor,
    const void* const* inputs, int num_inputs, void* const* outputs, int num_outputs, void* stream,
    int repeats, double* total_us);

/* TcExecutor::compiledSource, CudaTcExecutor::grid()/block() (cuda_tc_executor.h:52-60) */
const char* tc_executor_source(const tc_executor_t* executor);
int tc_executor_num_kernels(const tc_executor_t* executor);
int tc_executor_launch_bounds(const tc_executor_t* executor, int kernel, unsigned grid[3], unsigned block[3]);
const char* tc_executor_kernel_name(const tc_executor_t* executor, int kernel);
int64_t tc_executor_lds_bytes(const tc_executor_t* executor, int kernel);
/* CudaTcExecutor::clearRuntimeCompiledFunction (cuda_tc_executor.h:47-50) */
int tc_executor_clear(tc_executor_t* executor);
void tc_executor_destroy(tc_executor_t* executor);

/* Mapping options (CudaMappingOptions presets, tc/core/cuda/cuda_mapping_options.cc:327-384).
 * Presets: naive, single_thread, pointwise, mlp, conv, group_conv, unmapped. */
int tc_options_normalize(const char* options, char** text);          /* full "key=value;..." form */
int tc_options_to_serialized(const char* options, void** bytes, size_t* size);
int tc_options_from_serialized(const void* bytes, size_t size, char** text);
int tc_options_to_cpp(const char* options, char** cpp);              /* chainable C++ source */

/* The mapper alone: HIP source and launch bounds for the given shapes, nothing compiled or
 * loaded (what CudaBackend::compileWithTcMapper returns, cuda_tc_executor.cc:71-109). */
int tc_map(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs, const char* options,
    char** source, int* num_kernels, unsigned* grids /* [8][3] */, unsigned* blocks /* [8][3] */);

/* Front-end dumps in the format of the reference's golden files (tc/lang/test_expected/).
 * what: "lexer", "exp", "stmt", "function", "sema", "sema_env", "canonical"; and "ranges":
 * size-parametric range inference of one definition (tc/core/tc2halide.cc:270-498) — the bounds
 * of every tensor as expressions of the size parameters in the layout of the reference's
 * inference tests (test/test_inference.cc:28-67: "mins:" / "extents:" blocks, '//' for floor
 * division), followed by "statements:" with the range of every index variable. */
int tc_lang_dump(const char* text, const char* what, char** out);

/* ATenAutotuner<HipBackend, GeneticSearch>::tune (tc/aten/aten_autotuner.h:79-84,
 * tc/autotuner/autotuner.h:153-161).  Tensors must live on the current device; outputs are
 * scratch the candidates write into.  `settings` is "key=value;..." over generations, pop_size,
 * crossover_rate, mutation_rate, number_elites, threads, seed, cache_file, top_k,
 * min_launch_total_threads, max_serial_depth_ratio, seed_heuristics, refinement_rounds, resample_duplicates, fix_inert, fix_* ; NULL = flag
 * defaults.  Returns the best option text in *best (top_k best, newline separated). */
int tc_autotune(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const tc_dl_tensor* const* outputs, int num_outputs,
    const char* base_options, const char* settings, char** best);

/* The `count` best options recorded for this TC and these input sizes in an options cache file
 * written by a tuning run (`cache_file` setting); an empty text when the file or the entry is
 * missing.  loadTopKFromCacheFile, tc/autotuner/options_cache-inl.h:338-356, as used by
 * make_load_from_cache_options_factory (tensor_comprehensions/__init__.py:278-296). */
int tc_options_cache_load(
    const char* tc, const char* entry_point,
    const tc_dl_tensor* const* inputs, int num_inputs,
    const char* cache_file, int count, char** best);

/* Host-side tuner logic without a device, for bindings and tests:
 *   "powers2_and_ceil_divisors", "72"  -> "1,2,3,4,5,8,9,..."   (tc/autotuner/utils.cc:42-56)
 *   "search_space", "<shape>;<shape>..." e.g. "500x26x72;500x72x26" -> candidate value sets
 *   "options_cache_dump", "<file>" -> the entries of an options cache file as text, one per line:
 *       id | device | inputs | outputs | options | median runtime
 *   "median", "3,1,2,10" -> "2"                                  (tc/core/utils/math.h:23-37)
 *   "tuner_seeds", "<lowest output rank>[,<innermost output extent>]:<shape>;<shape>..." -> the structured starting points
 *       generation 0 holds next to the base mapping, one option text per line
 *   "sync_placement", "<cyclic 0|1>;<stages>;i:k:level,..." -> "position:level,..." (barriers the
 *       exact placement puts after stage `position` for the given stage-to-stage requirements) */
int tc_host_query(const char* what, const char* arg, char** out);

#ifdef __cplusplus
}
#endif
#endif /* TC_HIP_H */
