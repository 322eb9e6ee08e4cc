#include "tc/core/compiler.h"

#include <sstream>

#include <iostream>

#include "tc/core/check.h"
#include "tc/core/flags.h"
#include "tc/lang/parser.h"
#include "tc/lang/sema.h"

namespace tc {
namespace detail {

std::map<std::string, lang::TreeRef> parse(const std::string& tc) {
  lang::Parser parser(tc);
  std::map<std::string, lang::TreeRef> out;
  while (parser.L.cur().kind != lang::TK_EOF) {
    lang::TreeRef t = parser.parseFunction();
    if (flags().debug_lang) std::cerr << "[LANG] parsed definition:\n" << t << std::endl;
    out.emplace(lang::Def(t).name().name(), t);
  }
  return out;
}

ir::Function translate(
    const lang::TreeRef& def, const std::vector<const DLConstTensor*>& inputs, const CompilerOptions& options) {
  std::vector<std::vector<int64_t>> shapes;
  for (auto t : inputs) {
    shapes.emplace_back(t->shape, t->shape + t->ndim);
  }
  return tc2ir::translate(def, shapes, options);
}

namespace {
int scalarToken(uint8_t code, uint8_t bits) {
  return lang::TypeInfo(static_cast<lang::TypeInfo::Code>(code), bits).toScalarToken();
}
[[noreturn]] void throwInvalidStride(const lang::TreeRef& param, const DLConstTensor* t) {
  lang::ErrorReport e(param->range());
  std::ostringstream ss;
  ss << e.what() << "compilation aborted: invalid strides in tensor " << std::endl << *t << std::endl;
  throw InvalidStrideException(ss.str());
}
} // namespace

void checkInputsCompliant(const ir::Function& f, const std::vector<const DLConstTensor*>& inputs) {
  lang::Def def(f.def);
  if (inputs.size() != f.inputs.size()) {
    throw lang::errorAt(f.def) << "expected " << f.inputs.size() << " inputs but found " << inputs.size();
  }
  for (size_t i = 0; i < inputs.size(); ++i) {
    const DLConstTensor* t = inputs[i];
    const ir::Tensor& decl = f.inputs[i];
    int want = scalarToken(static_cast<uint8_t>(decl.type.code), static_cast<uint8_t>(decl.type.bits));
    int got = scalarToken(t->dtype.code, t->dtype.bits);
    // a bool tensor is a byte per element holding 0 or 1: DLPack's (uint, 8) stands for it as
    // well as the one-bit type the front end infers
    bool boolAsByte = decl.type.isBool() && t->dtype.code == kDLUInt && t->dtype.bits == 8;
    if (want != got && !boolAsByte) {
      throw lang::errorAt(def.params()[i]) << "expected type " << lang::kindToString(want) << " but found "
                                           << lang::kindToString(got);
    }
    if (t->ndim != static_cast<int>(decl.extents.size())) {
      throw lang::errorAt(def.params()[i]) << "expected a tensor with " << decl.extents.size()
                                           << " dimensions but found " << t->ndim << " dimensions.";
    }
    if (t->ndim > 0 && t->strides) {
      if (t->strides[t->ndim - 1] < 1) {
        throwInvalidStride(def.params()[i], t);
      }
      for (int j = 0; j + 1 < t->ndim; ++j) {
        if (t->strides[j] < t->strides[j + 1] * t->shape[j + 1]) {
          throwInvalidStride(def.params()[i], t);
        }
      }
    }
  }
}

std::vector<TensorInfo> inferOutputTensorInfo(
    const lang::TreeRef& def, const std::vector<const DLConstTensor*>& inputs, const CompilerOptions& options) {
  ir::Function f = translate(def, inputs, options);
  std::vector<TensorInfo> out;
  for (const auto& o : f.outputs) {
    out.emplace_back(o.type.toDL(), 0, o.extents, makeStridesFromSizes(o.extents));
  }
  return out;
}

} // namespace detail

std::vector<TensorInfo> inferOutputTensorInfo(
    const std::string& tc,
    const std::string& entryPoint,
    const std::vector<const DLConstTensor*>& inputs,
    const CompilerOptions& compilerOptions) {
  auto defs = detail::parse(tc);
  auto it = defs.find(entryPoint);
  if (it == defs.end()) {
    throw std::runtime_error("attempting to access undefined function " + entryPoint);
  }
  return detail::inferOutputTensorInfo(it->second, inputs, compilerOptions);
}

} // namespace tc
