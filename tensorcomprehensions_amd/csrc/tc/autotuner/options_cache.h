// Cache of tuned mapping options with their recorded runtimes.
//
// A multimap from (canonical TC text, input TensorInfos, output TensorInfos, backend string) to
// (options, recorded runtimes); ranking is by the median of all runtimes recorded for an option.
// Semantics follow the reference (tc/autotuner/options_cache.h:85-188, options_cache-inl.h:42-370);
// files use the wire format of tc/proto/compcache.proto:20-62 with the HIP options message as
// value.  Runtimes are stored in nanoseconds here (the reference stored whole microseconds).
#pragma once
#include <algorithm>
#include <fstream>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "tc/autotuner/utils.h"
#include "tc/core/tensor.h"
#include "tc/core/utils/protowire.h"
#include "tc/core/utils/time.h"

namespace tc {
namespace autotune {

struct OptionsCacheKey {
  std::string id; // canonical TC
  std::vector<TensorInfo> inputs, outputs;
  std::string backendStr;
  bool operator==(const OptionsCacheKey& o) const {
    return id == o.id && inputs == o.inputs && outputs == o.outputs && backendStr == o.backendStr;
  }
  bool operator<(const OptionsCacheKey& o) const {
    if (id != o.id) return id < o.id;
    if (backendStr != o.backendStr) return backendStr < o.backendStr;
    if (inputs != o.inputs) return inputs < o.inputs;
    return outputs < o.outputs;
  }
};

template <typename Backend>
struct OptionsCacheValue {
  typename Backend::MappingOptionsType mappingOptions;
  std::vector<Duration> runtimes;
};

template <typename Backend>
class OptionsCache {
 public:
  using Options = typename Backend::MappingOptionsType;
  using Value = OptionsCacheValue<Backend>;

  void clear() {
    std::lock_guard<std::mutex> lock(mutex_);
    store_.clear();
    numberCacheAttempts = numberAttemptedRetrievals = numberSuccessfulRetrievals = 0;
  }
  size_t size() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return store_.size();
  }
  size_t count(const OptionsCacheKey& key) const {
    std::lock_guard<std::mutex> lock(mutex_);
    return store_.count(key);
  }
  std::vector<OptionsCacheKey> getKeys() const {
    std::lock_guard<std::mutex> lock(mutex_);
    std::vector<OptionsCacheKey> keys;
    for (auto it = store_.begin(); it != store_.end(); it = store_.upper_bound(it->first)) {
      keys.push_back(it->first);
    }
    return keys;
  }

  // Appends the runtime to the entry holding the same options, or inserts a new entry.
  void recordRuntime(
      const std::string& canonicalTc, const std::vector<TensorInfo>& inputs, const std::vector<TensorInfo>& outputs,
      const std::string& backendStr, const Options& options, Duration duration) {
    std::lock_guard<std::mutex> lock(mutex_);
    ++numberCacheAttempts;
    OptionsCacheKey key{canonicalTc, inputs, outputs, backendStr};
    auto range = store_.equal_range(key);
    for (auto it = range.first; it != range.second; ++it) {
      if (it->second.mappingOptions == options) {
        it->second.runtimes.push_back(duration);
        return;
      }
    }
    store_.emplace(key, Value{options, {duration}});
  }

  std::vector<std::pair<Options, Duration>> getTopKEntries(
      const std::string& canonicalTc, const std::vector<TensorInfo>& inputs, const std::vector<TensorInfo>& outputs,
      const std::string& backendStr, size_t K) const {
    std::lock_guard<std::mutex> lock(mutex_);
    ++numberAttemptedRetrievals;
    OptionsCacheKey key{canonicalTc, inputs, outputs, backendStr};
    auto range = store_.equal_range(key);
    std::vector<std::pair<Options, Duration>> all;
    for (auto it = range.first; it != range.second; ++it) {
      all.emplace_back(it->second.mappingOptions, medianOf(it->second.runtimes));
    }
    if (all.empty()) return all;
    ++numberSuccessfulRetrievals;
    std::stable_sort(all.begin(), all.end(), [](const auto& a, const auto& b) { return a.second < b.second; });
    if (all.size() > K) all.resize(K);
    return all;
  }

  std::vector<Options> getTopKOptions(
      const std::string& canonicalTc, const std::vector<TensorInfo>& inputs, const std::vector<TensorInfo>& outputs,
      const std::string& backendStr, size_t K) const {
    std::vector<Options> out;
    for (auto& e : getTopKEntries(canonicalTc, inputs, outputs, backendStr, K)) out.push_back(e.first);
    return out;
  }

  // Keeps, for every key, the K options with the best median runtime.
  void pruneKeepTopK(size_t K) {
    std::lock_guard<std::mutex> lock(mutex_);
    std::multimap<OptionsCacheKey, Value> kept;
    for (auto it = store_.begin(); it != store_.end();) {
      auto end = store_.upper_bound(it->first);
      std::vector<const Value*> vals;
      for (auto j = it; j != end; ++j) vals.push_back(&j->second);
      std::stable_sort(vals.begin(), vals.end(), [](const Value* a, const Value* b) {
        return medianOf(a->runtimes) < medianOf(b->runtimes);
      });
      for (size_t i = 0; i < vals.size() && i < K; ++i) kept.emplace(it->first, *vals[i]);
      it = end;
    }
    store_.swap(kept);
  }

  std::string toProtobuf() const {
    std::lock_guard<std::mutex> lock(mutex_);
    protowire::Writer w;
    for (const auto& kv : store_) w.bytes(1, keyToProto(kv.first));
    for (const auto& kv : store_) {
      protowire::Writer v;
      v.bytes(1, kv.second.mappingOptions.toProtobufSerializedString());
      for (auto d : kv.second.runtimes) v.varint(2, static_cast<uint64_t>(d.toNanoSeconds()));
      w.bytes(2, v.str());
    }
    return w.str();
  }
  // Inserts every (key, value) pair of the message; duplicates are not merged.
  void fromProtobuf(const std::string& s) {
    std::vector<OptionsCacheKey> keys;
    std::vector<Value> values;
    protowire::Reader r(s);
    while (r.next()) {
      if (r.field() == 1) keys.push_back(keyFromProto(r.bytes()));
      if (r.field() == 2) {
        Value v;
        protowire::Reader vr(r.bytes());
        while (vr.next()) {
          if (vr.field() == 1) v.mappingOptions = Options(vr.bytes());
          if (vr.field() == 2) vr.eachValue([&](uint64_t ns) { v.runtimes.push_back(Duration::fromNanoSeconds(static_cast<int64_t>(ns))); });
        }
        values.push_back(std::move(v));
      }
    }
    if (keys.size() != values.size()) throw std::runtime_error("options cache: keys and values differ in number");
    std::lock_guard<std::mutex> lock(mutex_);
    for (size_t i = 0; i < keys.size(); ++i) store_.emplace(keys[i], values[i]);
  }

  void loadCacheFromFile(const std::string& filename) {
    std::ifstream in(filename, std::ios::binary);
    if (!in) throw std::runtime_error("cannot open options cache " + filename);
    std::string s((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    fromProtobuf(s);
  }
  void storeCacheToFile(const std::string& filename) const {
    std::string s = toProtobuf();
    std::ofstream out(filename, std::ios::binary | std::ios::trunc);
    if (!out) throw std::runtime_error("cannot write options cache " + filename);
    out.write(s.data(), static_cast<std::streamsize>(s.size()));
  }

  mutable size_t numberCacheAttempts = 0, numberAttemptedRetrievals = 0, numberSuccessfulRetrievals = 0;

 private:
  static Duration medianOf(const std::vector<Duration>& d) {
    std::vector<int64_t> ns;
    for (auto x : d) ns.push_back(x.toNanoSeconds());
    return Duration::fromNanoSeconds(median(ns));
  }
  static std::string tensorToProto(const TensorInfo& t) {
    protowire::Writer w;
    for (auto s : t.shape) w.varint(1, static_cast<uint64_t>(s));
    for (auto s : t.strides) w.varint(2, static_cast<uint64_t>(s));
    w.varint(3, t.alignment);
    protowire::Writer d;
    d.varint(1, t.dtype.code);
    d.varint(2, t.dtype.bits);
    d.varint(3, t.dtype.lanes);
    w.bytes(4, d.str());
    return w.str();
  }
  static TensorInfo tensorFromProto(const std::string& s) {
    TensorInfo t(DLDataType{2, 32, 1}, 0, {}, {});
    protowire::Reader r(s);
    while (r.next()) {
      if (r.field() == 1) r.eachValue([&](uint64_t e) { t.shape.push_back(static_cast<int64_t>(e)); });
      if (r.field() == 2) r.eachValue([&](uint64_t e) { t.strides.push_back(static_cast<int64_t>(e)); });
      if (r.field() == 3) t.alignment = r.value();
      if (r.field() == 4) {
        protowire::Reader d(r.bytes());
        while (d.next()) {
          if (d.field() == 1) t.dtype.code = static_cast<uint8_t>(d.value());
          if (d.field() == 2) t.dtype.bits = static_cast<uint8_t>(d.value());
          if (d.field() == 3) t.dtype.lanes = static_cast<uint16_t>(d.value());
        }
      }
    }
    return t;
  }
  static std::string keyToProto(const OptionsCacheKey& k) {
    protowire::Writer w;
    w.bytes(1, k.id);
    for (const auto& t : k.inputs) w.bytes(2, tensorToProto(t));
    for (const auto& t : k.outputs) w.bytes(3, tensorToProto(t));
    w.bytes(4, k.backendStr);
    w.bytes(5, "tc-hip");
    return w.str();
  }
  static OptionsCacheKey keyFromProto(const std::string& s) {
    OptionsCacheKey k;
    protowire::Reader r(s);
    while (r.next()) {
      if (r.field() == 1) k.id = r.bytes();
      if (r.field() == 2) k.inputs.push_back(tensorFromProto(r.bytes()));
      if (r.field() == 3) k.outputs.push_back(tensorFromProto(r.bytes()));
      if (r.field() == 4) k.backendStr = r.bytes();
    }
    return k;
  }

  mutable std::mutex mutex_;
  std::multimap<OptionsCacheKey, Value> store_;
};

// Best `count` options stored in `filename` for this problem; empty when the file is missing.
template <typename Backend>
std::vector<typename Backend::MappingOptionsType> loadTopKFromCacheFile(
    const std::string& canonicalTc, const std::vector<TensorInfo>& inputs, const std::vector<TensorInfo>& outputs,
    const std::string& filename, size_t count) {
  OptionsCache<Backend> cache;
  std::ifstream probe(filename);
  if (!probe) return {};
  cache.loadCacheFromFile(filename);
  return cache.getTopKOptions(canonicalTc, inputs, outputs, Backend::backendString(), count);
}

// Merges the best `count` options per key of `cache` into `filename` (created when missing).
template <typename Backend>
void appendTopKToCacheFile(const OptionsCache<Backend>& cache, const std::string& filename, size_t count) {
  OptionsCache<Backend> merged;
  std::ifstream probe(filename);
  if (probe) merged.loadCacheFromFile(filename);
  OptionsCache<Backend> copy;
  copy.fromProtobuf(cache.toProtobuf());
  copy.pruneKeepTopK(count);
  merged.fromProtobuf(copy.toProtobuf());
  merged.storeCacheToFile(filename);
}

} // namespace autotune
} // namespace tc
