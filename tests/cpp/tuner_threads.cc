// Host-side driver for a build of the library with ThreadSanitizer: the whole tuning loop (eight
// compile threads feeding the evaluation thread, outcomes shared between duplicate mappings, the
// options cache) runs against the cost model of tc/autotuner/model_backend.h.  No GPU call is
// made; a data race is reported on stderr and fails the run (halt_on_error).
#include <iostream>
#include <string>
#include "tc_hip.h"
#include "capi/tc_hip_testing.h"
int main() {
  const char* tcs[][3] = {
    {"moments", "1024x4096", "def moments(float(M, N) X) -> (mean, var) { mean(m) +=! X(m, r_n) / N\n var(m) +=! (X(m, r_n) - mean(m)) * (X(m, r_n) - mean(m)) / N }"},
    {"mm", "128x256;256x192", "def mm(float(M,K) A, float(K,N) B) -> (C) { C(m,n) +=! A(m,r_k) * B(r_k,n) }"},
    {"conv", "8x4x20x20;6x4x3x3", "def conv(float(N,C,H,W) I, float(F,C,KH,KW) W1) -> (O) { O(n,f,h,w) +=! I(n,c,h+kh,w+kw) * W1(f,c,kh,kw) }"}};
  for (auto& t : tcs) {
    for (int seed = 1; seed <= 3; ++seed) {
      std::string arg = "generations=4;pop_size=24;threads=8;seed=" + std::to_string(seed) + "|" + t[0] + "|" + t[1] + "|" + t[2];
      char* answer = nullptr;
      if (tc_testing_query("tune_on_model", arg.c_str(), &answer) != 0) { std::cerr << "failed: " << tc_last_error() << "\n"; return 1; }
      tc_free(answer);
    }
  }
  std::cout << "9 tunings done\n";
  return 0;
}
