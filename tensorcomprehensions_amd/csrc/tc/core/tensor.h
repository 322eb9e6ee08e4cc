// Tensor metadata crossing the compile / run boundary.
//
// DLTensor / DLConstTensor are laid out exactly like DLPack's C structs so a caller holding a
// DLPack tensor can pass its address through; tc::TensorInfo is the pointer-free description
// (dtype, alignment of the data pointer modulo 256, shape, strides) used as tuning-cache key.
// Counterpart of tc/core/tensor.h:27-140 and tc/core/tensor.cc:28-105.
#pragma once
#include <cstdint>
#include <memory>
#include <ostream>
#include <string>
#include <vector>

extern "C" {
typedef enum { kDLCPU = 1, kDLGPU = 2, kDLCPUPinned = 3, kDLROCM = 10 } DLDeviceType;
typedef struct {
  DLDeviceType device_type;
  int device_id;
} DLContext;
typedef enum { kDLInt = 0U, kDLUInt = 1U, kDLFloat = 2U } DLDataTypeCode;
typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;
typedef struct {
  void* data;
  DLContext ctx;
  int ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides;
  uint64_t byte_offset;
} DLTensor;
typedef struct {
  const void* data;
  DLContext ctx;
  int ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides;
  uint64_t byte_offset;
} DLConstTensor;
}

namespace tc {

// The unique_ptr owns shape/strides and the struct itself, never the data.
struct DLTensorDeleter {
  template <typename T>
  void operator()(const T* t) const {
    if (t) {
      delete[] t->shape;
      delete[] t->strides;
      delete t;
    }
  }
};
using DLTensorUPtr = std::unique_ptr<DLTensor, DLTensorDeleter>;
using DLConstTensorUPtr = std::unique_ptr<DLConstTensor, DLTensorDeleter>;

inline std::vector<int64_t> makeStridesFromSizes(const std::vector<int64_t>& sizes) {
  std::vector<int64_t> strides(sizes.size(), 1);
  for (int i = static_cast<int>(sizes.size()) - 2; i >= 0; --i) {
    strides[i] = strides[i + 1] * sizes[i + 1];
  }
  return strides;
}

struct TensorInfo {
  static constexpr int kAlignment = 256;
  DLDataType dtype;
  uint64_t alignment;
  std::vector<int64_t> shape;
  std::vector<int64_t> strides;

  TensorInfo(DLDataType d, uint64_t a, std::vector<int64_t> sh, std::vector<int64_t> st)
      : dtype(d), alignment(a), shape(std::move(sh)), strides(std::move(st)) {}
  template <typename DLT>
  static TensorInfo fromDL(const DLT* t) {
    std::vector<int64_t> sh(t->shape, t->shape + t->ndim);
    std::vector<int64_t> st = t->strides ? std::vector<int64_t>(t->strides, t->strides + t->ndim)
                                         : makeStridesFromSizes(sh);
    uint64_t addr = reinterpret_cast<uint64_t>(t->data) + t->byte_offset;
    return TensorInfo(t->dtype, addr % kAlignment, std::move(sh), std::move(st));
  }
  explicit TensorInfo(const DLTensor* t) : TensorInfo(fromDL(t)) {}
  explicit TensorInfo(const DLConstTensor* t) : TensorInfo(fromDL(t)) {}
  bool operator==(const TensorInfo& o) const {
    return dtype.code == o.dtype.code && dtype.bits == o.dtype.bits && dtype.lanes == o.dtype.lanes &&
        alignment == o.alignment && shape == o.shape && strides == o.strides;
  }
  bool operator!=(const TensorInfo& o) const { return !(*this == o); }
  bool operator<(const TensorInfo& o) const {
    if (shape != o.shape) return shape < o.shape;
    if (strides != o.strides) return strides < o.strides;
    if (alignment != o.alignment) return alignment < o.alignment;
    if (dtype.code != o.dtype.code) return dtype.code < o.dtype.code;
    return dtype.bits < o.dtype.bits;
  }
};

template <typename DLT>
std::unique_ptr<DLT, DLTensorDeleter> makeDLTensor(
    const TensorInfo& info, decltype(DLT::data) data = nullptr, DLDeviceType dev = kDLROCM, int devId = 0) {
  std::unique_ptr<DLT, DLTensorDeleter> t(new DLT);
  t->data = data;
  t->ctx = DLContext{dev, devId};
  t->ndim = static_cast<int>(info.shape.size());
  t->dtype = info.dtype;
  t->shape = new int64_t[info.shape.size() + 1];
  t->strides = new int64_t[info.shape.size() + 1];
  for (size_t i = 0; i < info.shape.size(); ++i) {
    t->shape[i] = info.shape[i];
    t->strides[i] = info.strides[i];
  }
  t->byte_offset = 0;
  return t;
}

template <typename UPtr>
auto extractRawPtrs(const std::vector<UPtr>& v) -> std::vector<const typename UPtr::element_type*> {
  std::vector<const typename UPtr::element_type*> out;
  for (const auto& p : v) {
    out.push_back(p.get());
  }
  return out;
}

inline std::vector<TensorInfo> makeTensorInfoVector(const std::vector<const DLConstTensor*>& ts) {
  std::vector<TensorInfo> out;
  for (auto t : ts) {
    out.emplace_back(t);
  }
  return out;
}
inline std::vector<TensorInfo> makeTensorInfoVector(const std::vector<const DLTensor*>& ts) {
  std::vector<TensorInfo> out;
  for (auto t : ts) {
    out.emplace_back(t);
  }
  return out;
}

inline std::string toString(const DLDataType& t) {
  const char* base = t.code == kDLFloat ? "float" : t.code == kDLInt ? "int" : "uint";
  return std::string(base) + std::to_string(static_cast<int>(t.bits));
}

inline std::ostream& operator<<(std::ostream& os, const TensorInfo& t) {
  os << toString(t.dtype) << " align " << t.alignment << " sizes [";
  for (size_t i = 0; i < t.shape.size(); ++i) {
    os << (i ? ", " : "") << t.shape[i];
  }
  os << "] strides [";
  for (size_t i = 0; i < t.strides.size(); ++i) {
    os << (i ? ", " : "") << t.strides[i];
  }
  return os << "]";
}
template <typename DLT>
inline std::ostream& printDL(std::ostream& os, const DLT& t) {
  return os << TensorInfo::fromDL(&t);
}
inline std::ostream& operator<<(std::ostream& os, const DLTensor& t) { return printDL(os, t); }
inline std::ostream& operator<<(std::ostream& os, const DLConstTensor& t) { return printDL(os, t); }

// Thrown when an input's strides are not monotone / dense enough for the generated indexing.
struct InvalidStrideException : public std::runtime_error {
  explicit InvalidStrideException(const std::string& s) : std::runtime_error(s) {}
};

} // namespace tc
