// Helpers shared by the translation units that implement the C ABI.
#pragma once
#include <string>
#include <vector>

#include "tc/core/tensor.h"
#include "tc_hip.h"

namespace tc {
namespace capi {
extern thread_local std::string lastError;
char* dupString(const std::string& s);
std::vector<const DLConstTensor*> constTensors(const tc_dl_tensor* const* ts, int n);
std::vector<const DLTensor*> mutTensors(const tc_dl_tensor* const* ts, int n);
} // namespace capi
} // namespace tc
