// at::Tensor <-> DLTensor glue: metadata-owning DLTensor views over ATen tensors.
// Counterpart of tc/aten/aten.h and tc/aten/aten-inl.h:60-104 (the reference goes through
// at::toDLPack; here the DLPack-layout structs are filled directly, data is never owned).
#pragma once
#include <ATen/ATen.h>

#include <vector>

#include "tc/core/check.h"
#include "tc/core/tensor.h"

namespace tc {
namespace aten {

inline DLDataType toDLDataType(const at::Tensor& t) {
  DLDataType d;
  d.lanes = 1;
  d.bits = static_cast<uint8_t>(t.element_size() * 8);
  switch (t.scalar_type()) {
    case at::kFloat: case at::kDouble: case at::kHalf: d.code = kDLFloat; break;
    case at::kByte: case at::kBool: case at::kUInt16: case at::kUInt32: case at::kUInt64: d.code = kDLUInt; break;
    case at::kChar: case at::kShort: case at::kInt: case at::kLong: d.code = kDLInt; break;
    default: TC_CHECK(false) << "unsupported ATen scalar type";
  }
  return d;
}

inline at::ScalarType toScalarType(const DLDataType& d) {
  if (d.code == kDLFloat) return d.bits == 64 ? at::kDouble : d.bits == 16 ? at::kHalf : at::kFloat;
  if (d.code == kDLUInt) {
    // (a TC `bool` is an 8-bit unsigned value on the device, like uint8)
    return d.bits == 64 ? at::kUInt64 : d.bits == 32 ? at::kUInt32 : d.bits == 16 ? at::kUInt16 : at::kByte;
  }
  switch (d.bits) {
    case 8: return at::kChar;
    case 16: return at::kShort;
    case 32: return at::kInt;
    default: return at::kLong;
  }
}

template <typename DLT>
std::unique_ptr<DLT, DLTensorDeleter> makeDLView(const at::Tensor& t) {
  std::vector<int64_t> shape(t.sizes().begin(), t.sizes().end()), strides(t.strides().begin(), t.strides().end());
  TensorInfo info(toDLDataType(t), 0, shape, strides);
  return makeDLTensor<DLT>(
      info, t.data_ptr(), t.is_cuda() ? kDLROCM : kDLCPU, t.is_cuda() ? static_cast<int>(t.get_device()) : 0);
}

inline std::vector<DLConstTensorUPtr> makeDLConstTensors(const std::vector<at::Tensor>& ts) {
  std::vector<DLConstTensorUPtr> out;
  for (const auto& t : ts) out.push_back(makeDLView<DLConstTensor>(t));
  return out;
}
inline std::vector<DLTensorUPtr> makeDLTensors(const std::vector<at::Tensor>& ts) {
  std::vector<DLTensorUPtr> out;
  for (const auto& t : ts) out.push_back(makeDLView<DLTensor>(t));
  return out;
}

} // namespace aten
} // namespace tc
