// Genetic search over TuningConfigurations.
//
// Same algorithm as the reference (tc/autotuner/genetic_search.h:51-111, genetic_search.cc:30-310):
// the population starts from the given configurations plus random valid ones; after every
// generation invalid candidates are dropped, the rest sorted by runtime, parents are drawn by
// roulette wheel on 1/runtime, children come from a three-parent uniform crossover (with
// probability crossOverRate %) or are copies of one selected parent, and all non-elite members
// are mutated gene by gene with probability mutationRate %.  With fewer than three valid
// candidates the population is re-randomised around the last best configuration.
#pragma once
#include <memory>
#include <random>
#include <vector>

#include "tc/autotuner/parameters.h"

namespace tc {
namespace autotune {

class GeneticSearch {
 public:
  using Population = std::vector<std::unique_ptr<CandidateConfiguration>>;

  // seed < 0: seeded from std::random_device (non-deterministic, as the reference by default)
  GeneticSearch(
      const std::vector<TuningConfiguration>& confs,
      size_t numGenerations,
      size_t populationSize,
      uint8_t crossOverRate,
      uint8_t mutationRate,
      size_t numElites,
      int64_t seed = -1);

  // Requires a recorded runtime on every valid candidate; produces the next generation.
  void updateParameters();

  // Mutates one candidate once more (deviation: the autotuner calls it for bred candidates that
  // would repeat a mapping it has measured).
  void remutate(CandidateConfiguration& candidate) { mutate(candidate); }

  Population population;
  TuningConfiguration lastBestConf;
  const size_t numGenerations;
  const size_t maxPopulationSize;
  const uint8_t crossOverRate;
  const uint8_t mutationRate;
  const size_t numberElites;
  static constexpr int mutateIterations = 1000;
  static constexpr size_t minCandidatesForBreeding = 3;

 private:
  TuningConfiguration crossover(TuningConfiguration& a, TuningConfiguration& b, TuningConfiguration& c);
  void breed();
  void randomize(Population::iterator begin, Population::iterator end);
  void mutate(CandidateConfiguration& c);
  std::mt19937_64 rng_;
};

} // namespace autotune
} // namespace tc
