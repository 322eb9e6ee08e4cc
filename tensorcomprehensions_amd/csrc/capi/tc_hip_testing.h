/* C ABI of libtc_hip_testing.so: host-side test scaffolding kept out of the product library.
 * Strings are returned as in tc_hip.h (release with tc_free_string, errors through tc_last_error). */
#ifndef TC_HIP_TESTING_H
#define TC_HIP_TESTING_H
#ifdef __cplusplus
extern "C" {
#endif
/*   "genetic_search", "seed=..;generations=..;pop_size=.." -> best synthetic cost per generation
 *   "tune_on_model", "<settings>|<entry point>|<shape>;<shape>...|<tc text>" -> the whole tune() against the
 *       cost model of tc/autotuner/model_backend.h: "best=<options>\ncost_ns=..\nnaive_ns=.."
 *   "options_cache_selftest", "<scratch file>" -> "name=value" lines: what a sample cache answers (sizes,
 *       ranking by median, misses, pruning, wire and file round trips; test/cuda/test_compilation_cache.cc:133-510)
 *   "options_cache_write_sample", "<file>" -> stores that sample cache (compcache.proto wire format) and
 *       returns its entries as text, one per line
 *   "base_outside_space", "" -> how the tuner answers a base mapping outside its candidate values */
int tc_testing_query(const char* what, const char* arg, char** out);
#ifdef __cplusplus
}
#endif
#endif /* TC_HIP_TESTING_H */
