// Small numeric helpers of the tuner (counterpart of tc/autotuner/utils.h, tc/core/utils/math.h).
#pragma once
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <vector>

namespace tc {
namespace autotune {

// {1, 2, 4, ..., 2^ceil(log2(val))}
inline std::vector<size_t> powers2(size_t val) {
  std::vector<size_t> r;
  size_t p = 1;
  r.push_back(p);
  while (p < val) {
    p *= 2;
    r.push_back(p);
  }
  return r;
}

// powers2(val) plus ceil(val / p) for every power p <= val, sorted, unique.
// Known answers: tc::autotune tests (test/cuda/test_autotuner_utility.cc:34-50).
inline std::vector<size_t> powers2andCeilDivisors(size_t val) {
  std::vector<size_t> r = powers2(val);
  size_t n = r.size();
  for (size_t i = 0; i < n; ++i) {
    if (r[i] <= val) {
      r.push_back((val + r[i] - 1) / r[i]);
    }
  }
  std::sort(r.begin(), r.end());
  r.erase(std::unique(r.begin(), r.end()), r.end());
  return r;
}

template <typename T>
std::vector<T> mergeVectors(std::vector<T> a, const std::vector<T>& b) {
  a.insert(a.end(), b.begin(), b.end());
  std::sort(a.begin(), a.end());
  a.erase(std::unique(a.begin(), a.end()), a.end());
  return a;
}

// Median; for an even count the mean of the two middle values (tc/core/utils/math.h:23-37).
template <typename T>
T median(std::vector<T> v) {
  std::sort(v.begin(), v.end());
  size_t n = v.size();
  if (n == 0) {
    return T();
  }
  return n % 2 ? v[n / 2] : (v[n / 2 - 1] + v[n / 2]) / 2;
}

} // namespace autotune
} // namespace tc
