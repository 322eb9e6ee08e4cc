// tc_autotune: C ABI of the genetic autotuner.
#include "capi/tc_capi_internal.h"

extern "C" int tc_autotune(
    const char*, const char*, const tc_dl_tensor* const*, int, const tc_dl_tensor* const*, int,
    const char*, const char*, char**) {
  tc::capi::lastError = "autotuner not linked into this build";
  return 1;
}
