// Durations and profiling results.
//
// The reference stores std::chrono::microseconds (tc/core/utils/time.h:21-80), which rounds a
// sub-microsecond kernel to 0 and makes the tuner discard it (tc/autotuner/autotuner-inl.h:199-201).
// Kernels on this hardware routinely run for a few microseconds, so Duration keeps nanoseconds
// and exposes the same accessors plus fractional ones.
#pragma once
#include <chrono>
#include <cstdint>
#include <limits>
#include <ostream>

namespace tc {

class Duration {
 public:
  Duration() : ns_(0) {}
  static Duration fromNanoSeconds(int64_t ns) {
    Duration d;
    d.ns_ = ns;
    return d;
  }
  static Duration fromMicroSeconds(double us) { return fromNanoSeconds(static_cast<int64_t>(us * 1e3 + 0.5)); }
  static Duration zero() { return Duration(); }
  static Duration max() { return fromNanoSeconds(std::numeric_limits<int64_t>::max()); }
  template <typename Clock>
  static Duration since(std::chrono::time_point<Clock> t0) {
    return fromNanoSeconds(std::chrono::duration_cast<std::chrono::nanoseconds>(Clock::now() - t0).count());
  }
  int64_t toNanoSeconds() const { return ns_; }
  int64_t toMicroSeconds() const { return ns_ / 1000; }
  double toMicroSecondsF() const { return ns_ / 1e3; }
  Duration operator+(Duration o) const { return fromNanoSeconds(ns_ + o.ns_); }
  Duration operator-(Duration o) const { return fromNanoSeconds(ns_ - o.ns_); }
  Duration operator*(int64_t k) const { return fromNanoSeconds(ns_ * k); }
  Duration operator/(int64_t k) const { return fromNanoSeconds(ns_ / k); }
  bool operator<(Duration o) const { return ns_ < o.ns_; }
  bool operator<=(Duration o) const { return ns_ <= o.ns_; }
  bool operator>(Duration o) const { return ns_ > o.ns_; }
  bool operator>=(Duration o) const { return ns_ >= o.ns_; }
  bool operator==(Duration o) const { return ns_ == o.ns_; }
  bool operator!=(Duration o) const { return ns_ != o.ns_; }

 private:
  int64_t ns_;
};

inline std::ostream& operator<<(std::ostream& os, Duration d) {
  return os << d.toMicroSecondsF() << "us";
}

struct ProfilingInfo {
  Duration cpuOverhead;
  Duration kernelRuntime;
};

} // namespace tc
