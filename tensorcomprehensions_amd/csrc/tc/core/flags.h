// Process-wide knobs.  Names and defaults mirror the reference's gflags (tc/core/flags.cc:24-130);
// here they are plain globals, optionally overridden from the environment as TC_<NAME>.
#pragma once
#include <cstdint>
#include <string>

namespace tc {
struct Flags {
  bool debug_lang = false;           // print every parsed definition (its tree) to stderr
  bool debug_tc_mapper = false;      // print the options and the launches the mapper decided on
  bool debug_tuner = false;
  bool dump_hip = false;             // print generated HIP source at compile time
  bool fast_math = false;            // pass -ffast-math to hipRTC (the reference used --use_fast_math)
  // (benchmark_warmup / benchmark_iterations of flags.cc:59-66 steer the reference's benchmark
  // fixture, not its library: here they are bench.py's --warmup / --steps, which read the
  // environment variables TC_BENCHMARK_WARMUP / TC_BENCHMARK_ITERATIONS for their defaults.
  // tuner_gen_restore_from_proto of flags.cc:107-110 has no reader in the reference either: a
  // cache file is named per tuning run, TunerSettings::cacheFile.)
  // tuner (flags.cc:77-122)
  uint32_t tuner_gen_pop_size = 100;
  uint32_t tuner_gen_crossover_rate = 80;
  uint32_t tuner_gen_mutation_rate = 7;
  uint32_t tuner_gen_generations = 25;
  uint32_t tuner_gen_number_elites = 10;
  uint32_t tuner_threads = 8;
  std::string tuner_devices = "0";   // comma-separated; candidates are measured on the first that holds the tensors
  uint32_t tuner_gen_restore_number = 10;
  bool tuner_gen_log_generations = false;
  uint64_t tuner_min_launch_total_threads = 64;
  std::string tuner_rng_restore;
  int64_t random_seed = -1;
};
Flags& flags();
// Seed shared by host-side random choices: flags().random_seed if >= 0, else time-derived,
// always reduced modulo 15485863 (flags.cc:132-144).
uint64_t initRandomSeed();
const uint64_t& randomSeed();
} // namespace tc
