// Size-parametric range inference: the ranges of every index variable and the bounds of every
// tensor of a TC definition as expressions of the size parameters named in its signature,
// without knowing the sizes.
//
// The reference infers ranges on Halide expressions over the size parameters and specialises
// them later (tc/core/tc2halide.cc:270-498, halide_utils.cc:41-86, polyhedral/scop.h:110-124);
// its known answers (test/test_inference.cc:70-540) are such expressions.  The compile pipeline
// of this library infers on the concrete sizes of a call (tc2ir.cc); this file restates the same
// solver on symbolic bounds for callers that want shapes before they have tensors: an output's
// extents as formulas, evaluated for any sizes afterwards (FunctionRanges::evaluate).
//
// Bounds are linear forms over atoms; an atom is a size parameter or a floor-division, minimum
// or maximum of linear forms that does not simplify.  Texts use '//' for floor division, so a
// bound prints as an expression Python evaluates as it stands.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "tc/lang/tree.h"
#include "tc/utils/compiler_options.h"

namespace tc {
namespace symbolic {

struct Lin {
  std::map<std::string, int64_t> coef; // atom key -> coefficient (never 0)
  int64_t k = 0;
  bool isConstant() const { return coef.empty(); }
};

struct Atom {
  enum Kind { Param, FloorDiv, Min, Max } kind = Param;
  Lin a, b;       // FloorDiv: a // d;  Min/Max: of a and b
  int64_t d = 1;
};

struct Range { // inclusive
  Lin min, max;
};

struct TensorBounds {
  std::string name;
  std::vector<Lin> mins, extents;
};

struct StatementRanges {
  std::string tensor;
  std::vector<std::pair<std::string, Range>> vars; // left-hand indices, then reduction indices
};

struct FunctionRanges {
  std::string name;
  std::vector<std::string> params;       // size parameters in order of first appearance
  std::vector<TensorBounds> inputs, outputs;
  std::vector<StatementRanges> statements;
  std::map<std::string, Atom> atoms;

  std::string text(const Lin& e) const;
  int64_t evaluate(const Lin& e, const std::map<std::string, int64_t>& sizes) const;
  // "mins:\n<tensor>@[..; ]\n...extents:\n..." in the layout of the reference's inference tests
  std::string dump() const;
};

// Throws lang::ErrorReport where the concrete inference would for any sizes (unsolved variables,
// non-integer range bounds); what depends on the sizes (empty ranges, accesses out of bounds for
// part of a range) is not diagnosed here.
FunctionRanges inferRanges(const lang::TreeRef& def, const CompilerOptions& options);

} // namespace symbolic
} // namespace tc
