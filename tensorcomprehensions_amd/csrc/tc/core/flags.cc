#include "tc/core/flags.h"

#include <cstdlib>
#include <ctime>
#include <mutex>

namespace tc {
namespace {
void envU32(const char* name, uint32_t* v) {
  if (const char* e = std::getenv(name)) *v = static_cast<uint32_t>(std::strtoul(e, nullptr, 10));
}
void envBool(const char* name, bool* v) {
  if (const char* e = std::getenv(name)) *v = e[0] == '1' || e[0] == 't' || e[0] == 'T';
}
uint64_t g_seed = static_cast<uint64_t>(-1);
} // namespace

Flags& flags() {
  static Flags f = [] {
    Flags x;
    envBool("TC_DEBUG_LANG", &x.debug_lang);
    envBool("TC_DEBUG_TC_MAPPER", &x.debug_tc_mapper);
    envBool("TC_DEBUG_TUNER", &x.debug_tuner);
    envBool("TC_DUMP_HIP", &x.dump_hip);
    envBool("TC_FAST_MATH", &x.fast_math);
    envU32("TC_TUNER_GEN_POP_SIZE", &x.tuner_gen_pop_size);
    envU32("TC_TUNER_GEN_CROSSOVER_RATE", &x.tuner_gen_crossover_rate);
    envU32("TC_TUNER_GEN_MUTATION_RATE", &x.tuner_gen_mutation_rate);
    envU32("TC_TUNER_GEN_GENERATIONS", &x.tuner_gen_generations);
    envU32("TC_TUNER_GEN_NUMBER_ELITES", &x.tuner_gen_number_elites);
    envU32("TC_TUNER_THREADS", &x.tuner_threads);
    if (const char* e = std::getenv("TC_TUNER_DEVICES")) x.tuner_devices = e;
    envU32("TC_TUNER_GEN_RESTORE_NUMBER", &x.tuner_gen_restore_number);
    envBool("TC_TUNER_GEN_LOG_GENERATIONS", &x.tuner_gen_log_generations);
    if (const char* e = std::getenv("TC_TUNER_RNG_RESTORE")) x.tuner_rng_restore = e;
    if (const char* e = std::getenv("TC_RANDOM_SEED")) x.random_seed = std::strtoll(e, nullptr, 10);
    return x;
  }();
  return f;
}

uint64_t initRandomSeed() {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  if (g_seed == static_cast<uint64_t>(-1)) {
    g_seed = flags().random_seed >= 0 ? static_cast<uint64_t>(flags().random_seed) : static_cast<uint64_t>(std::time(nullptr));
    g_seed %= 15485863ULL;
  }
  return g_seed;
}
const uint64_t& randomSeed() {
  initRandomSeed();
  return g_seed;
}
} // namespace tc
