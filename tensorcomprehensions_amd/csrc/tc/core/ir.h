// The front end's output: a TC function specialised on concrete input sizes.
//
// This small IR takes the place the Halide statements take in the reference
// (tc/core/tc2halide.h:29-61 HalideComponents).  After semantic analysis and range inference
// every statement is `lhs(idx...) op= expr` over a rectangular box of index values, which is
// all the mapper needs; size parameters are already substituted by their values.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "tc/core/tensor.h"
#include "tc/lang/tree.h"
#include "tc/utils/compiler_options.h"

namespace tc {
namespace ir {

struct ScalarType {
  enum Code { Int = 0, UInt = 1, Float = 2 };
  Code code = Float;
  int bits = 32;
  bool isFloat() const { return code == Float; }
  bool isBool() const { return code == UInt && bits == 1; }
  bool operator==(const ScalarType& o) const { return code == o.code && bits == o.bits; }
  bool operator!=(const ScalarType& o) const { return !(*this == o); }
  int bytes() const { return bits <= 8 ? 1 : bits / 8; }
  // spelling in generated device / host C
  std::string cName() const {
    if (code == Float) {
      return bits == 64 ? "double" : bits == 16 ? "_Float16" : "float";
    }
    if (isBool()) {
      return "bool";
    }
    // (plain `char` has no fixed signedness: int8 is spelled out)
    return std::string(code == UInt ? "unsigned " : bits == 8 ? "signed " : "") +
        (bits == 8 ? "char" : bits == 16 ? "short" : bits == 32 ? "int" : "long long");
  }
  DLDataType toDL() const {
    return DLDataType{static_cast<uint8_t>(code), static_cast<uint8_t>(isBool() ? 8 : bits), 1};
  }
};

struct Expr;
using ExprRef = std::shared_ptr<const Expr>;

struct Expr {
  enum Kind { IntImm, FloatImm, Var, Load, Binary, Unary, Select, Cast, Call };
  Kind kind;
  ScalarType type;
  int64_t ival = 0;      // IntImm
  double fval = 0;       // FloatImm
  std::string name;      // Var: index; Load: tensor; Call: function; Binary/Unary: operator
  std::vector<ExprRef> args;
};

// Inclusive interval of index values.
struct Range {
  int64_t min = 0, max = -1;
  int64_t extent() const { return max - min + 1; }
};

// coef . vars + constant, or invalid when the subscript is not integer-affine in the indices
struct Affine {
  bool valid = false;
  std::map<std::string, int64_t> coef;
  int64_t constant = 0;
  int64_t coefOf(const std::string& v) const {
    auto it = coef.find(v);
    return it == coef.end() ? 0 : it->second;
  }
};
Affine toAffine(const ExprRef& e);

enum class ReduceOp { None, Plus, Times, Min, Max };

struct Statement {
  std::string tensor;                   // written tensor
  std::vector<std::string> lhsVars;     // its subscripts, all plain index variables
  std::vector<std::string> redVars;     // reduction indices, first-appearance order
  std::map<std::string, Range> ranges;  // every index above
  ReduceOp op = ReduceOp::None;         // None: plain assignment
  bool init = false;                    // "op=!": start from the operator's identity
  ExprRef rhs;
  ScalarType type;
  lang::TreeRef tree;                   // for error reports
  // Set by the mapper when it divides a sum among blocks: `sliceVar` (the first of lhsVars, not a
  // subscript of the tensor) numbers the slices of the outermost reduction index, and the
  // partial result of a slice is added into the tensor atomically.  `zeroing` marks the statement
  // that clears the tensor beforehand: it is mapped as a plain fill, whatever the options say
  // about tiles and blocks (their positions mean the variables of the sliced statement).
  bool atomic = false;
  bool zeroing = false;
  std::string sliceVar;
};

struct Tensor {
  std::string name;
  ScalarType type;
  std::vector<int64_t> mins, extents;
  std::vector<std::string> argNames;    // index names of the defining statement (outputs)
  bool isInput = false;
  std::vector<int64_t> strides() const { return makeStridesFromSizes(extents); }
  int64_t numel() const {
    int64_t n = 1;
    for (auto e : extents) {
      n *= e;
    }
    return n;
  }
};

struct Function {
  std::string name;
  std::vector<Tensor> inputs, outputs;
  std::map<std::string, int64_t> params;   // size variables, sorted by name
  std::vector<Statement> statements;
  std::vector<std::string> warnings;
  lang::TreeRef def;                        // checked tree
  const Tensor* find(const std::string& n) const {
    for (const auto& t : inputs) {
      if (t.name == n) return &t;
    }
    for (const auto& t : outputs) {
      if (t.name == n) return &t;
    }
    return nullptr;
  }
};

// Identity element of a reduction as a C literal of the given type (0, 1, type max, type min).
std::string identityLiteral(ReduceOp op, const ScalarType& t);

} // namespace ir

// Parse-tree -> IR.  `inputs` supplies the concrete shapes (and is checked against the declared
// ranks, constant dims and repeated size names).  Counterpart of tc2halide::translate
// (tc/core/tc2halide.cc:758-920) + computeParamValueMap (tc/core/halide_utils.cc:41-86).
namespace tc2ir {
ir::Function translate(
    const lang::TreeRef& def,
    const std::vector<std::vector<int64_t>>& inputShapes,
    const CompilerOptions& options = CompilerOptions());
} // namespace tc2ir
} // namespace tc
