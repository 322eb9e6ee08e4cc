#include "tc/autotuner/genetic_search.h"

#include <algorithm>
#include <numeric>
#include <sstream>

#include "tc/core/check.h"
#include "tc/core/flags.h"

namespace tc {
namespace autotune {

namespace {
template <typename RNG>
void randomizeParameter(RangeParameter& p, RNG& rng) {
  size_t n = p.numberOptions();
  p.selectOption(std::uniform_int_distribution<size_t>(0, n - 1)(rng));
}
} // namespace

GeneticSearch::GeneticSearch(
    const std::vector<TuningConfiguration>& confs,
    size_t numGenerations,
    size_t populationSize,
    uint8_t crossOverRate,
    uint8_t mutationRate,
    size_t numElites,
    int64_t seed)
    : lastBestConf(confs.at(0)),
      numGenerations(numGenerations),
      maxPopulationSize(populationSize),
      crossOverRate(crossOverRate),
      mutationRate(mutationRate),
      numberElites(std::min(numElites, populationSize / 2)),
      rng_(seed >= 0 ? static_cast<uint64_t>(seed) : std::random_device{}()) {
  if (!flags().tuner_rng_restore.empty()) {
    std::istringstream ss(flags().tuner_rng_restore);
    ss >> rng_;
  }
  TC_CHECK_LT(numberElites, maxPopulationSize);
  TC_CHECK(mutationRate <= 100) << "the mutation rate (" << int(mutationRate) << ") should be in the [0,100] interval";
  TC_CHECK(crossOverRate <= 100) << "the crossover (" << int(crossOverRate) << ") rate should be in the [0,100] interval";
  TC_CHECK(!confs.empty()) << "empty set of predefined configurations";
  population.reserve(populationSize);
  size_t size = 0;
  for (; size < confs.size() && size < maxPopulationSize; ++size) {
    population.emplace_back(new CandidateConfiguration(confs[size]));
  }
  size_t given = size;
  for (; size < maxPopulationSize; ++size) {
    population.emplace_back(new CandidateConfiguration(population.front()->configuration));
  }
  randomize(population.begin() + given, population.end());
}

void GeneticSearch::randomize(Population::iterator begin, Population::iterator end) {
  for (auto it = begin; it != end; ++it) {
    auto& conf = (*it)->configuration;
    do {
      conf.applyToParameters([&](RangeParameter& p) { randomizeParameter(p, rng_); });
    } while (!conf.isValid());
  }
}

void GeneticSearch::mutate(CandidateConfiguration& candidate) {
  std::discrete_distribution<int> should{static_cast<double>(100 - mutationRate), static_cast<double>(mutationRate)};
  for (int i = 0; i < mutateIterations; ++i) {
    TuningConfiguration res = candidate.configuration;
    res.applyToParameters([&](RangeParameter& p) {
      if (!p.isForced() && should(rng_)) randomizeParameter(p, rng_);
    });
    if (res.isValid()) {
      candidate.configuration = res;
      return;
    }
  }
}

TuningConfiguration GeneticSearch::crossover(TuningConfiguration& a, TuningConfiguration& b, TuningConfiguration& c) {
  auto pa = a.collectParameters(), pb = b.collectParameters(), pc = c.collectParameters();
  for (int iter = 0; iter < mutateIterations; ++iter) {
    TuningConfiguration child = a;
    auto params = child.collectParameters();
    for (size_t i = 0; i < params.size(); ++i) {
      switch (std::uniform_int_distribution<size_t>{0, 2}(rng_)) {
        case 0: *params[i] = *pa[i]; break;
        case 1: *params[i] = *pb[i]; break;
        default: *params[i] = *pc[i]; break;
      }
    }
    if (child.isValid()) {
      return child;
    }
  }
  return a;
}

void GeneticSearch::breed() {
  // accumulated, normalised fitness = 1 / runtime
  std::vector<double> acc;
  double sum = 0;
  for (const auto& c : population) sum += 1.0 / c->runtime.toMicroSecondsF();
  double run = 0;
  for (const auto& c : population) {
    run += (1.0 / c->runtime.toMicroSecondsF()) / sum;
    acc.push_back(run);
  }
  Population next;
  next.reserve(maxPopulationSize);
  for (const auto& p : population) {
    next.emplace_back(new CandidateConfiguration(p->configuration));
  }
  auto select = [&]() -> TuningConfiguration& {
    double limit = std::uniform_real_distribution<double>{}(rng_);
    size_t i = static_cast<size_t>(std::lower_bound(acc.begin(), acc.end(), limit) - acc.begin());
    return population.at(std::min(i, population.size() - 1))->configuration;
  };
  std::discrete_distribution<int> cross{static_cast<double>(100 - crossOverRate), static_cast<double>(crossOverRate)};
  while (next.size() < maxPopulationSize) {
    if (cross(rng_)) {
      TuningConfiguration p1 = select(), p2 = select(), p3 = select();
      next.emplace_back(new CandidateConfiguration(crossover(p1, p2, p3)));
    } else {
      next.emplace_back(new CandidateConfiguration(select()));
    }
  }
  population = std::move(next);
}

void GeneticSearch::updateParameters() {
  population.erase(
      std::remove_if(population.begin(), population.end(), [](const auto& c) { return c->invalid; }),
      population.end());
  for (const auto& c : population) {
    if (c->runtime == Duration::zero()) {
      throw std::invalid_argument(
          "All candidates must have a recorded runtime before the new parameters can be computed.");
    }
  }
  std::sort(population.begin(), population.end(), [](const auto& a, const auto& b) { return a->runtime < b->runtime; });
  if (!population.empty()) {
    lastBestConf = population.front()->configuration;
  }
  if (population.size() < minCandidatesForBreeding) {
    // too few survivors: restart around the last best configuration, keeping it as member 0
    population.clear();
    for (size_t i = 0; i < maxPopulationSize; ++i) {
      population.emplace_back(new CandidateConfiguration(lastBestConf));
    }
    randomize(population.begin() + 1, population.end());
    return;
  }
  breed();
  for (size_t i = numberElites; i < population.size(); ++i) {
    mutate(*population[i]);
  }
}

} // namespace autotune
} // namespace tc
