// Mapping options of the HIP backend for CDNA4.
//
// Same surface as the reference's CudaMappingOptions (tc/core/cuda/cuda_mapping_options.h:36-245,
// presets tc/core/cuda/cuda_mapping_options.cc:327-384, wire fields
// tc/proto/mapping_options.proto:74-96): grid, block, shared (LDS) and private (register)
// promotion switches and depths.  Differences, all motivated by the hardware:
//   * presets use blocks that are multiples of the 64-lane wavefront,
//   * extra fields (numbers 11+ on the wire): vectorWidth (adjacent elements per thread along the
//     contiguous dimension), collapseContiguous (merge loop dimensions that are jointly contiguous
//     in every tensor before mapping), useMfma (matrix-core tiles for dense contractions),
//     prefetchShared (software-pipelined LDS staging: the next block tile's global loads are
//     in flight while the current one is computed), reductionBlocks (a sum whose outermost
//     reduction index is divided among that many blocks, which add their partial results into
//     the output with atomics; 1 = the reference's behaviour, a reduction stays inside a block).
#pragma once
#include <algorithm>
#include <array>

#include "tc/core/mapping_options.h"

namespace tc {

// 1 to 3 strictly positive extents (x, then optional y, z).
class HipDim {
 public:
  HipDim() : v_{1} {}
  HipDim(std::initializer_list<uint64_t> l) : v_(l) { check(); }
  explicit HipDim(std::vector<uint64_t> v) : v_(std::move(v)) { check(); }
  size_t size() const { return v_.size(); }
  uint64_t operator[](size_t i) const { return i < v_.size() ? v_[i] : 1; }
  const std::vector<uint64_t>& extractVector() const { return v_; }
  std::array<uint64_t, 3> extractDefaultedArray() const { return {{(*this)[0], (*this)[1], (*this)[2]}}; }
  bool operator==(const HipDim& o) const { return v_ == o.v_; }
  std::string toCommaSeparatedString() const {
    std::string s;
    for (size_t i = 0; i < v_.size(); ++i) {
      s += (i ? ", " : "") + std::to_string(v_[i]);
    }
    return s;
  }
  std::string toProto() const {
    protowire::Writer w;
    for (size_t i = 0; i < v_.size(); ++i) w.varint(static_cast<int>(i) + 1, v_[i]);
    return w.str();
  }
  void fromProto(const std::string& s) {
    v_.clear();
    protowire::Reader r(s);
    while (r.next()) {
      if (r.field() >= 1 && r.field() <= 3) {
        v_.resize(std::max<size_t>(v_.size(), r.field()), 1);
        v_[r.field() - 1] = r.value();
      }
    }
    check();
  }

 private:
  void check() const {
    TC_CHECK_GE(v_.size(), 1u) << "need at least one mapping size";
    TC_CHECK_LE(v_.size(), 3u) << "at most three mapping sizes";
  }
  std::vector<uint64_t> v_;
};
using HipGrid = HipDim;
using HipBlock = HipDim;

class HipMappingOptions : public GenericOptionsFluent<HipMappingOptions> {
 public:
  MappingOptions generic;
  HipBlock block{64, 4};
  HipGrid grid{256, 256};
  bool useSharedMemoryValue = false;
  bool usePrivateMemoryValue = false;
  bool unrollCopySharedValue = false;
  bool hasMaxSharedMemory = false;
  uint64_t maxSharedMemoryValue = 0;
  bool useReadOnlyCacheValue = false;
  bool hasPrivateDepth = false;
  uint32_t privateDepthValue = 0;
  bool hasSharedDepth = false;
  uint32_t sharedDepthValue = 0;
  // CDNA4 extras
  uint32_t vectorWidthValue = 1;
  bool collapseContiguousValue = true;
  bool useMfmaValue = false;
  bool prefetchSharedValue = false;
  uint32_t reductionBlocksValue = 1;

  HipMappingOptions() = default;
  // from a serialized HipMappingOptionsProto
  explicit HipMappingOptions(const std::string& serialized) { fromProto(serialized); }

  bool operator==(const HipMappingOptions& o) const {
    return generic == o.generic && block == o.block && grid == o.grid &&
        useSharedMemoryValue == o.useSharedMemoryValue && usePrivateMemoryValue == o.usePrivateMemoryValue &&
        unrollCopySharedValue == o.unrollCopySharedValue && hasMaxSharedMemory == o.hasMaxSharedMemory &&
        (!hasMaxSharedMemory || maxSharedMemoryValue == o.maxSharedMemoryValue) &&
        useReadOnlyCacheValue == o.useReadOnlyCacheValue && privateDepthValue == o.privateDepthValue &&
        sharedDepthValue == o.sharedDepthValue && vectorWidthValue == o.vectorWidthValue &&
        collapseContiguousValue == o.collapseContiguousValue && useMfmaValue == o.useMfmaValue &&
        prefetchSharedValue == o.prefetchSharedValue && reductionBlocksValue == o.reductionBlocksValue;
  }
  bool operator!=(const HipMappingOptions& o) const { return !(*this == o); }

  HipMappingOptions& genericMappingOptions(const MappingOptions& g) {
    generic = g;
    return *this;
  }
  HipMappingOptions& mapToThreads(const std::vector<uint64_t>& v) {
    block = HipBlock(v);
    return *this;
  }
  HipMappingOptions& mapToThreads(std::initializer_list<uint64_t> l) { return mapToThreads(std::vector<uint64_t>(l)); }
  HipMappingOptions& mapToThreads(uint64_t x) { return mapToThreads(std::vector<uint64_t>{x}); }
  HipMappingOptions& mapToThreads(uint64_t x, uint64_t y) { return mapToThreads(std::vector<uint64_t>{x, y}); }
  HipMappingOptions& mapToThreads(uint64_t x, uint64_t y, uint64_t z) {
    return mapToThreads(std::vector<uint64_t>{x, y, z});
  }
  HipMappingOptions& mapToThreads(const std::string& csv) { return mapToThreads(parseCsv(csv)); }
  HipMappingOptions& mapToBlocks(const std::vector<uint64_t>& v) {
    grid = HipGrid(v);
    return *this;
  }
  HipMappingOptions& mapToBlocks(std::initializer_list<uint64_t> l) { return mapToBlocks(std::vector<uint64_t>(l)); }
  HipMappingOptions& mapToBlocks(uint64_t x) { return mapToBlocks(std::vector<uint64_t>{x}); }
  HipMappingOptions& mapToBlocks(uint64_t x, uint64_t y) { return mapToBlocks(std::vector<uint64_t>{x, y}); }
  HipMappingOptions& mapToBlocks(uint64_t x, uint64_t y, uint64_t z) {
    return mapToBlocks(std::vector<uint64_t>{x, y, z});
  }
  HipMappingOptions& mapToBlocks(const std::string& csv) { return mapToBlocks(parseCsv(csv)); }
  HipMappingOptions& useSharedMemory(bool b) { useSharedMemoryValue = b; return *this; }
  HipMappingOptions& usePrivateMemory(bool b) { usePrivateMemoryValue = b; return *this; }
  HipMappingOptions& unrollCopyShared(bool b) { unrollCopySharedValue = b; return *this; }
  HipMappingOptions& maxSharedMemory(uint64_t bytes) {
    hasMaxSharedMemory = true;
    maxSharedMemoryValue = bytes;
    return *this;
  }
  HipMappingOptions& useReadOnlyCache(bool b) { useReadOnlyCacheValue = b; return *this; }
  HipMappingOptions& privateDepth(uint32_t d) { hasPrivateDepth = true; privateDepthValue = d; return *this; }
  HipMappingOptions& sharedDepth(uint32_t d) { hasSharedDepth = true; sharedDepthValue = d; return *this; }
  HipMappingOptions& vectorWidth(uint32_t w) {
    TC_CHECK(w == 1 || w == 2 || w == 4) << "vector width must be 1, 2 or 4, got " << w;
    vectorWidthValue = w;
    return *this;
  }
  HipMappingOptions& collapseContiguous(bool b) { collapseContiguousValue = b; return *this; }
  HipMappingOptions& useMfma(bool b) { useMfmaValue = b; return *this; }
  HipMappingOptions& prefetchShared(bool b) { prefetchSharedValue = b; return *this; }
  HipMappingOptions& reductionBlocks(uint32_t n) {
    TC_CHECK(n >= 1 && n <= 1024) << "reductionBlocks must be between 1 and 1024, got " << n;
    reductionBlocksValue = n;
    return *this;
  }

  std::string toProtobufSerializedString() const {
    protowire::Writer w;
    w.bytes(1, generic.toProto());
    w.bytes(2, block.toProto());
    w.bytes(3, grid.toProto());
    w.boolean(4, useSharedMemoryValue);
    w.boolean(5, usePrivateMemoryValue);
    w.boolean(6, unrollCopySharedValue);
    if (hasMaxSharedMemory) w.varint(7, maxSharedMemoryValue);
    w.boolean(8, useReadOnlyCacheValue);
    if (hasPrivateDepth) w.varint(9, privateDepthValue);
    if (hasSharedDepth) w.varint(10, sharedDepthValue);
    w.varint(11, vectorWidthValue);
    w.boolean(12, collapseContiguousValue);
    w.boolean(13, useMfmaValue);
    w.boolean(14, prefetchSharedValue);
    if (reductionBlocksValue != 1) w.varint(15, reductionBlocksValue);
    return w.str();
  }
  void fromProto(const std::string& s) {
    protowire::Reader r(s);
    while (r.next()) {
      switch (r.field()) {
        case 1: generic.fromProto(r.bytes()); break;
        case 2: block.fromProto(r.bytes()); break;
        case 3: grid.fromProto(r.bytes()); break;
        case 4: useSharedMemoryValue = r.value() != 0; break;
        case 5: usePrivateMemoryValue = r.value() != 0; break;
        case 6: unrollCopySharedValue = r.value() != 0; break;
        case 7: hasMaxSharedMemory = true; maxSharedMemoryValue = r.value(); break;
        case 8: useReadOnlyCacheValue = r.value() != 0; break;
        case 9: hasPrivateDepth = true; privateDepthValue = static_cast<uint32_t>(r.value()); break;
        case 10: hasSharedDepth = true; sharedDepthValue = static_cast<uint32_t>(r.value()); break;
        // (through the setters: a foreign or damaged file must not plant a value the text form refuses)
        case 11: vectorWidth(static_cast<uint32_t>(std::min<uint64_t>(r.value(), 1u << 20))); break;
        case 12: collapseContiguousValue = r.value() != 0; break;
        case 13: useMfmaValue = r.value() != 0; break;
        case 14: prefetchSharedValue = r.value() != 0; break;
        case 15: reductionBlocks(static_cast<uint32_t>(std::min<uint64_t>(r.value(), 1u << 20))); break;
        default: break;
      }
    }
  }

  // Presets.  Tile sizes / unroll / fusion as in the reference presets; thread blocks re-shaped
  // to whole 64-lane wavefronts with x (the contiguous dimension) 64 wide.
  static HipMappingOptions makeUnmappedMappingOptions() {
    HipMappingOptions o;
    o.generic = MappingOptions::makeUnmappedMappingOptions();
    o.block = HipBlock{1};
    o.grid = HipGrid{1};
    return o;
  }
  static HipMappingOptions makeNaiveMappingOptions() {
    return makeUnmappedMappingOptions().tile(32, 32, 32).mapToThreads(64, 4).mapToBlocks(256, 256).unroll(1);
  }
  static HipMappingOptions makeSingleThreadMappingOptions() {
    return makeUnmappedMappingOptions().tile(1).mapToThreads(1).mapToBlocks(1).unroll(1);
  }
  static HipMappingOptions makePointwiseMappingOptions() {
    return makeUnmappedMappingOptions().tile(32, 32, 32).mapToThreads(64, 2, 2).mapToBlocks(100, 100, 100).unroll(128);
  }
  static HipMappingOptions makeMlpMappingOptions() {
    return makeUnmappedMappingOptions()
        .outerScheduleFusionStrategy(FusionStrategy::Max)
        .tile(1)
        .mapToThreads(128)
        .mapToBlocks(128)
        .unroll(1);
  }
  static HipMappingOptions makeConvolutionMappingOptions() {
    return makeUnmappedMappingOptions().tile(4, 8, 8, 8).mapToThreads(8, 8, 4).mapToBlocks(256, 256, 256).unroll(1);
  }
  static HipMappingOptions makeGroupConvolutionMappingOptions() {
    return makeUnmappedMappingOptions().tile(1, 1).mapToThreads(8, 8, 4).mapToBlocks(256, 256).unroll(1);
  }

  // "key=value;..." text used by the C ABI and the Python layer.
  std::string toText() const;
  static HipMappingOptions fromText(const std::string& text);

 private:
  static std::vector<uint64_t> parseCsv(const std::string& csv) {
    std::vector<uint64_t> v;
    std::stringstream ss(csv);
    std::string item;
    while (std::getline(ss, item, ',')) {
      if (!item.empty()) v.push_back(std::stoull(item));
    }
    return v;
  }
};

std::ostream& operator<<(std::ostream& os, const HipMappingOptions& o);

// Prints options as chainable C++ (what a user pastes back into code); layout follows the
// reference printers (tc/core/mapping_options_cpp_printer.cc:37-58,
// tc/core/cuda/cuda_mapping_options_cpp_printer.cc:22-46).
class HipMappingOptionsAsCpp {
 public:
  explicit HipMappingOptionsAsCpp(const HipMappingOptions& o, size_t indent = 0) : options(o), indent(indent) {}
  const HipMappingOptions& options;
  size_t indent;
};
std::ostream& operator<<(std::ostream& os, const HipMappingOptionsAsCpp& o);

// Stream wrapper with the reference printer's calling convention
// (`HipMappingOptionsCppPrinter(out, indent) << options`,
// tc/core/cuda/cuda_mapping_options_cpp_printer.h:34-46).
class HipMappingOptionsCppPrinter {
 public:
  explicit HipMappingOptionsCppPrinter(std::ostream& out, size_t ws = 0) : out_(out), ws_(ws) {}
  friend HipMappingOptionsCppPrinter& operator<<(HipMappingOptionsCppPrinter& prn, const HipMappingOptions& options) {
    prn.out_ << HipMappingOptionsAsCpp(options, prn.ws_);
    return prn;
  }

 private:
  std::ostream& out_;
  size_t ws_;
};

} // namespace tc
