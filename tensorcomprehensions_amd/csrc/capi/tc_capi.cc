// C ABI over the C++ library (declared in include/tc_hip.h).  Exceptions stop here: each entry
// point catches, stores the message per thread and returns a non-zero status.
#include "tc/core/symbolic_ranges.h"
#include "tc_hip.h"

#include <cstdlib>
#include <cstring>
#include <iostream>
#include <mutex>
#include <set>
#include <sstream>

#include "capi/tc_capi_internal.h"
#include "tc/core/compiler.h"
#include "tc/core/hip/hip_tc_executor.h"
#include "tc/lang/parser.h"
#include "tc/lang/sema.h"

static_assert(sizeof(tc_dl_tensor) == sizeof(DLTensor), "tc_dl_tensor must match the DLPack layout");
static_assert(sizeof(tc_dl_tensor) == sizeof(DLConstTensor), "tc_dl_tensor must match the DLPack layout");

struct tc_executor {
  std::unique_ptr<tc::HipTcExecutor> impl;
};

namespace tc {
namespace capi {
thread_local std::string lastError;
thread_local tc::CompilerOptions compilerOptions;

char* dupString(const std::string& s) {
  char* p = static_cast<char*>(std::malloc(s.size() + 1));
  std::memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

std::vector<const DLConstTensor*> constTensors(const tc_dl_tensor* const* ts, int n) {
  std::vector<const DLConstTensor*> v;
  for (int i = 0; i < n; ++i) v.push_back(reinterpret_cast<const DLConstTensor*>(ts[i]));
  return v;
}
std::vector<const DLTensor*> mutTensors(const tc_dl_tensor* const* ts, int n) {
  std::vector<const DLTensor*> v;
  for (int i = 0; i < n; ++i) v.push_back(reinterpret_cast<const DLTensor*>(ts[i]));
  return v;
}
} // namespace capi
} // namespace tc

using namespace tc::capi;

#define TC_CAPI_BEGIN try {
#define TC_CAPI_END                      \
  }                                      \
  catch (const std::exception& e) {      \
    lastError = e.what();                \
    return 1;                            \
  }                                      \
  catch (...) {                          \
    lastError = "unknown C++ exception"; \
    return 2;                            \
  }                                      \
  return 0;

extern "C" {

const char* tc_last_error(void) {
  return lastError.c_str();
}
void tc_free(void* p) {
  std::free(p);
}
void tc_set_compiler_options(int emitWarnings, int throwWarnings) {
  compilerOptions.emitWarnings = emitWarnings != 0;
  compilerOptions.throwWarnings = throwWarnings != 0;
}

int tc_infer_output_info(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    tc_tensor_info* outputs, int capacity, int* count) {
  TC_CAPI_BEGIN
  auto infos = tc::inferOutputTensorInfo(tcText, entry, constTensors(inputs, numInputs), compilerOptions);
  *count = static_cast<int>(infos.size());
  for (int i = 0; i < *count && i < capacity; ++i) {
    const tc::TensorInfo& t = infos[i];
    TC_CHECK_LE(t.shape.size(), static_cast<size_t>(TC_MAX_RANK)) << "output rank too large for tc_tensor_info";
    outputs[i].dtype = tc_dl_datatype{t.dtype.code, t.dtype.bits, t.dtype.lanes};
    outputs[i].ndim = static_cast<int32_t>(t.shape.size());
    for (size_t d = 0; d < t.shape.size(); ++d) {
      outputs[i].shape[d] = t.shape[d];
      outputs[i].strides[d] = t.strides[d];
    }
  }
  TC_CAPI_END
}

int tc_compile(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    const char* options, tc_executor_t** executor) {
  TC_CAPI_BEGIN
  auto opts = tc::HipMappingOptions::fromText(options ? options : "naive");
  auto ex = tc::compile<tc::HipBackend>(tcText, entry, constTensors(inputs, numInputs), opts, compilerOptions);
  *executor = new tc_executor{std::move(ex)};
  TC_CAPI_END
}

int tc_compile_serialized_options(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    const void* options, size_t optionsSize, tc_executor_t** executor) {
  TC_CAPI_BEGIN
  tc::HipMappingOptions opts(std::string(static_cast<const char*>(options), optionsSize));
  auto ex = tc::compile<tc::HipBackend>(tcText, entry, constTensors(inputs, numInputs), opts, compilerOptions);
  *executor = new tc_executor{std::move(ex)};
  TC_CAPI_END
}

int tc_executor_run(
    const tc_executor_t* ex, const tc_dl_tensor* const* inputs, int numInputs,
    const tc_dl_tensor* const* outputs, int numOutputs, void* stream) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  tc::HipRuntimeInformation info;
  info.stream = stream;
  ex->impl->run(constTensors(inputs, numInputs), mutTensors(outputs, numOutputs), info);
  TC_CAPI_END
}

int tc_executor_unchecked_run(
    const tc_executor_t* ex, const void* const* inputs, int numInputs, void* const* outputs,
    int numOutputs, void* stream) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  tc::HipRuntimeInformation info;
  info.stream = stream;
  ex->impl->uncheckedRun(
      std::vector<const void*>(inputs, inputs + numInputs), std::vector<void*>(outputs, outputs + numOutputs), info);
  TC_CAPI_END
}

int tc_executor_profile(
    const tc_executor_t* ex, const tc_dl_tensor* const* inputs, int numInputs,
    const tc_dl_tensor* const* outputs, int numOutputs, void* stream, double* kernelUs, double* cpuUs) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  tc::HipRuntimeInformation info;
  info.stream = stream;
  tc::ProfilingInfo pi = ex->impl->profile(constTensors(inputs, numInputs), mutTensors(outputs, numOutputs), info);
  if (kernelUs) *kernelUs = pi.kernelRuntime.toMicroSecondsF();
  if (cpuUs) *cpuUs = pi.cpuOverhead.toMicroSecondsF();
  TC_CAPI_END
}

int tc_executor_profile_repeated(
    const tc_executor_t* ex, const void* const* inputs, int numInputs, void* const* outputs, int numOutputs,
    void* stream, int repeats, double* totalUs) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  tc::HipRuntimeInformation info;
  info.stream = stream;
  tc::Duration d = ex->impl->profileRepeated(
      std::vector<const void*>(inputs, inputs + numInputs), std::vector<void*>(outputs, outputs + numOutputs), repeats, info);
  *totalUs = d.toMicroSecondsF();
  TC_CAPI_END
}

const char* tc_executor_source(const tc_executor_t* ex) {
  return ex && ex->impl ? ex->impl->compiledSource.c_str() : "";
}
int tc_executor_num_kernels(const tc_executor_t* ex) {
  return ex && ex->impl ? static_cast<int>(ex->impl->compilationResult().kernels.size()) : 0;
}
int tc_executor_launch_bounds(const tc_executor_t* ex, int kernel, unsigned grid[3], unsigned block[3]) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  const auto& k = ex->impl->compilationResult().kernels.at(kernel);
  for (int a = 0; a < 3; ++a) {
    grid[a] = k.grid[a];
    block[a] = k.block[a];
  }
  TC_CAPI_END
}
const char* tc_executor_kernel_name(const tc_executor_t* ex, int kernel) {
  if (!ex || !ex->impl || kernel < 0 || kernel >= tc_executor_num_kernels(ex)) return "";
  return ex->impl->compilationResult().kernels[kernel].name.c_str();
}
int64_t tc_executor_lds_bytes(const tc_executor_t* ex, int kernel) {
  if (!ex || !ex->impl || kernel < 0 || kernel >= tc_executor_num_kernels(ex)) return -1;
  return ex->impl->compilationResult().program.kernels[kernel].ldsBytes;
}
int tc_executor_clear(tc_executor_t* ex) {
  TC_CAPI_BEGIN
  TC_CHECK(ex && ex->impl) << "null executor";
  ex->impl->clearRuntimeCompiledFunction();
  TC_CAPI_END
}
void tc_executor_destroy(tc_executor_t* ex) {
  delete ex;
}

int tc_options_normalize(const char* options, char** text) {
  TC_CAPI_BEGIN
  const std::string given = options ? options : "naive";
  *text = dupString(tc::HipMappingOptions::fromText(given).toText());
  // Options that steer the reference's isl scheduler or its promotion depth and that the box
  // mapper gives no meaning to are accepted, stored and round-tripped; naming one gets a note on
  // stderr, once per option and process.
  static std::mutex mu;
  static std::set<std::string> noted;
  for (const char* key : {"fixParametersBeforeScheduling", "tileImperfectlyNested", "privateDepth", "outerScheduleAllowSkewing",
                          "outerSchedulePositiveOrthant", "intraTileScheduleAllowSkewing", "intraTileSchedulePositiveOrthant"}) {
    if (given.find(std::string(key) + "=") == std::string::npos) continue;
    std::lock_guard<std::mutex> lock(mu);
    if (noted.insert(key).second) {
      std::cerr << "note: mapping option '" << key << "' is kept for compatibility with the reference's options and does not "
                << "change the mapping of this backend\n";
    }
  }
  TC_CAPI_END
}
int tc_options_to_serialized(const char* options, void** bytes, size_t* size) {
  TC_CAPI_BEGIN
  std::string s = tc::HipMappingOptions::fromText(options ? options : "naive").toProtobufSerializedString();
  *bytes = std::malloc(s.size() + 1);
  std::memcpy(*bytes, s.data(), s.size());
  *size = s.size();
  TC_CAPI_END
}
int tc_options_from_serialized(const void* bytes, size_t size, char** text) {
  TC_CAPI_BEGIN
  tc::HipMappingOptions o(std::string(static_cast<const char*>(bytes), size));
  *text = dupString(o.toText());
  TC_CAPI_END
}
int tc_options_to_cpp(const char* options, char** cpp) {
  TC_CAPI_BEGIN
  std::ostringstream ss;
  ss << tc::HipMappingOptionsAsCpp(tc::HipMappingOptions::fromText(options ? options : "naive"));
  *cpp = dupString(ss.str());
  TC_CAPI_END
}

int tc_map(
    const char* tcText, const char* entry, const tc_dl_tensor* const* inputs, int numInputs,
    const char* options, char** source, int* numKernels, unsigned* grids, unsigned* blocks) {
  TC_CAPI_BEGIN
  auto defs = tc::detail::parse(tcText);
  auto it = defs.find(entry);
  TC_CHECK(it != defs.end()) << "attempting to access undefined function " << entry;
  auto in = constTensors(inputs, numInputs);
  tc::ir::Function f = tc::detail::translate(it->second, in, compilerOptions);
  tc::detail::checkInputsCompliant(f, in);
  auto r = tc::HipBackend::compileWithTcMapper(
      f.name, f, in, tc::HipMappingOptions::fromText(options ? options : "naive"));
  *source = dupString(r.source);
  *numKernels = static_cast<int>(r.kernels.size());
  for (size_t k = 0; k < r.kernels.size() && k < 8; ++k) {
    for (int a = 0; a < 3; ++a) {
      if (grids) grids[k * 3 + a] = r.kernels[k].grid[a];
      if (blocks) blocks[k * 3 + a] = r.kernels[k].block[a];
    }
  }
  TC_CAPI_END
}

int tc_lang_dump(const char* text, const char* what, char** out) {
  TC_CAPI_BEGIN
  std::string w = what;
  std::ostringstream ss;
  if (w == "lexer") {
    lang::Lexer lex(text);
    while (lex.cur().kind != lang::TK_EOF) {
      ss << "FOUND '" << lang::kindToString(lex.cur().kind) << "'\n";
      lex.cur().range.highlight(ss);
      ss << "---------\n";
      lex.next();
    }
  } else if (w == "exp") {
    ss << lang::Parser(text).parseExp();
  } else if (w == "stmt") {
    ss << lang::Parser(text).parseStmt();
  } else if (w == "function") {
    ss << lang::Parser(text).parseFunction();
  } else if (w == "sema" || w == "sema_env" || w == "sema+env") {
    lang::Sema sema(compilerOptions);
    lang::TreeRef r = sema.checkFunction(lang::Parser(text).parseFunction());
    if (w != "sema_env") ss << r;
    if (w != "sema") ss << sema.dumpEnv();
  } else if (w == "canonical") {
    tc::CompilerOptions quiet;
    quiet.emitWarnings = false;
    ss << lang::canonicalize(lang::Sema(quiet).checkFunction(lang::Parser(text).parseFunction()));
  } else if (w == "ranges") {
    // size-parametric range inference: tensor bounds in the layout of the reference's inference
    // tests (test/test_inference.cc:28-67), then the ranges of every statement's variables
    tc::symbolic::FunctionRanges r = tc::symbolic::inferRanges(lang::Parser(text).parseFunction(), compilerOptions);
    ss << r.dump() << "statements:\n";
    for (const auto& st : r.statements) {
      ss << st.tensor << ":";
      for (const auto& v : st.vars) ss << " " << v.first << " in [" << r.text(v.second.min) << ", " << r.text(v.second.max) << "];";
      ss << "\n";
    }
  } else {
    TC_CHECK(false) << "unknown dump kind " << w;
  }
  *out = dupString(ss.str());
  TC_CAPI_END
}

} // extern "C"
