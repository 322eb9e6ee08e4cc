// S-expression trees for the TC front end, typed accessors over them, and the dump format.
//
// A node is either an atom (number, string, bool) or a compound (kind + children + source
// range).  The shape of every compound (which child means what) and the pretty-printer's
// 40-column folding rule are fixed by the reference's golden dumps
// (tc/lang/test_expected/*.expected, produced through tc/lang/tree.h:185-231 and the node
// layouts in tc/lang/tree_views.h:191-510); the canonical dump doubles as the tuning-cache key.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <ostream>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "tc/lang/lexer.h"

namespace lang {

class Tree;
using TreeRef = std::shared_ptr<Tree>;
using TreeList = std::vector<TreeRef>;

class Tree : public std::enable_shared_from_this<Tree> {
 public:
  // atoms
  static TreeRef number(double v) {
    auto t = std::shared_ptr<Tree>(new Tree(TK_NUMBER));
    t->num_ = v;
    return t;
  }
  static TreeRef string(const std::string& s) {
    auto t = std::shared_ptr<Tree>(new Tree(TK_STRING));
    t->str_ = s;
    return t;
  }
  // compound; its range is widened to cover all non-atom children
  static TreeRef make(int kind, const SourceRange& r, TreeList children = {}) {
    auto t = std::shared_ptr<Tree>(new Tree(kind));
    size_t s = r.start(), e = r.end();
    for (const auto& c : children) {
      if (!c->isAtom()) {
        s = std::min(s, c->range().start());
        e = std::max(e, c->range().end());
      }
    }
    t->range_.reset(new SourceRange(r.file_ptr(), s, e));
    t->trees_ = std::move(children);
    return t;
  }

  int kind() const { return kind_; }
  bool isAtom() const { return !range_; }
  const SourceRange& range() const {
    if (!range_) {
      throw std::runtime_error("atoms have no source range");
    }
    return *range_;
  }
  double doubleValue() const {
    if (kind_ != TK_NUMBER) {
      throw std::runtime_error("not a number");
    }
    return num_;
  }
  const std::string& stringValue() const {
    if (kind_ != TK_STRING) {
      throw std::runtime_error("not a string");
    }
    return str_;
  }
  const TreeList& trees() const { return trees_; }
  const TreeRef& tree(size_t i) const { return trees_.at(i); }

  // Rebuilds a compound with fn applied to every child; atoms map to themselves.
  TreeRef map(const std::function<TreeRef(TreeRef)>& fn) {
    if (isAtom()) {
      return shared_from_this();
    }
    TreeList out;
    for (const auto& c : trees_) {
      out.push_back(fn(c));
    }
    return make(kind_, *range_, std::move(out));
  }
  void expect(int k, size_t n) const {
    if (kind_ != k || trees_.size() != n) {
      std::stringstream ss;
      ss << "expected kind '" << kindToString(k) << "' with " << n << " subtrees but found '"
         << kindToString(kind_) << "' with " << trees_.size() << " subtrees.\n";
      if (range_) {
        range_->highlight(ss);
      }
      throw std::runtime_error(ss.str());
    }
  }

 private:
  explicit Tree(int k) : kind_(k) {}
  int kind_;
  double num_ = 0;
  std::string str_;
  std::unique_ptr<SourceRange> range_;
  TreeList trees_;
};

// ---- dump ---------------------------------------------------------------------------------
inline void flatDump(std::ostream& out, const TreeRef& t) {
  if (t->kind() == TK_NUMBER) {
    out << t->doubleValue();
  } else if (t->kind() == TK_STRING) {
    out << t->stringValue();
  } else {
    out << "(" << kindToString(t->kind());
    for (const auto& c : t->trees()) {
      out << " ";
      flatDump(out, c);
    }
    out << ")";
  }
}

// A subtree is printed on one line when indent + its flat length stays under `col`,
// otherwise its children go on lines of their own, two spaces deeper.
inline void prettyDump(std::ostream& out, const TreeRef& t, size_t indent, size_t col = 40) {
  std::ostringstream flat;
  flatDump(flat, t);
  if (t->isAtom() || indent + flat.str().size() < col) {
    out << flat.str();
    return;
  }
  out << "(" << kindToString(t->kind());
  for (const auto& c : t->trees()) {
    out << "\n" << std::string(indent + 2, ' ');
    prettyDump(out, c, indent + 2, col);
  }
  out << ")";
}

inline std::ostream& operator<<(std::ostream& out, const TreeRef& t) {
  prettyDump(out, t, 0);
  return out << std::endl;
}

inline ErrorReport errorAt(const TreeRef& t) {
  return ErrorReport(t->range());
}

// ---- typed views ----------------------------------------------------------------------------
// Thin wrappers: each checks kind/arity on construction and names the children.
struct View {
  View(TreeRef t, int kind, size_t n) : tree_(std::move(t)) { tree_->expect(kind, n); }
  explicit View(TreeRef t) : tree_(std::move(t)) {}
  const TreeRef& ref() const { return tree_; }
  operator TreeRef() const { return tree_; }
  const SourceRange& range() const { return tree_->range(); }
  TreeRef tree_;
};

inline TreeRef makeList(const SourceRange& r, TreeList l = {}) {
  return Tree::make(TK_LIST, r, std::move(l));
}

struct Ident : View {
  explicit Ident(TreeRef t) : View(std::move(t), TK_IDENT, 1) {}
  const std::string& name() const { return tree_->tree(0)->stringValue(); }
  static TreeRef create(const SourceRange& r, const std::string& name) {
    return Tree::make(TK_IDENT, r, {Tree::string(name)});
  }
};

struct Apply : View { // (apply name (list args...)); TK_ACCESS shares the layout
  explicit Apply(TreeRef t) : View(std::move(t)) {
    if (tree_->kind() != TK_APPLY && tree_->kind() != TK_ACCESS) {
      tree_->expect(TK_APPLY, 2);
    }
  }
  Ident name() const { return Ident(tree_->tree(0)); }
  const TreeList& arguments() const { return tree_->tree(1)->trees(); }
  TreeRef argumentList() const { return tree_->tree(1); }
  static TreeRef create(int kind, const SourceRange& r, TreeRef name, TreeRef args) {
    return Tree::make(kind, r, {std::move(name), std::move(args)});
  }
};

struct BuiltIn : View { // (built-in name (list args...) type)
  explicit BuiltIn(TreeRef t) : View(std::move(t), TK_BUILT_IN, 3) {}
  const std::string& name() const { return tree_->tree(0)->stringValue(); }
  const TreeList& arguments() const { return tree_->tree(1)->trees(); }
  TreeRef type() const { return tree_->tree(2); }
  static TreeRef create(const SourceRange& r, const std::string& name, TreeRef args, TreeRef type) {
    return Tree::make(TK_BUILT_IN, r, {Tree::string(name), std::move(args), std::move(type)});
  }
};

struct TensorType : View { // (tensor_type scalar (list dims...))
  explicit TensorType(TreeRef t) : View(std::move(t), TK_TENSOR_TYPE, 2) {}
  TreeRef scalarTypeTree() const { return tree_->tree(0); }
  int scalarType() const { return tree_->tree(0)->kind(); }
  const TreeList& dims() const { return tree_->tree(1)->trees(); }
  static TreeRef create(const SourceRange& r, TreeRef scalar, TreeRef dims) {
    return Tree::make(TK_TENSOR_TYPE, r, {std::move(scalar), std::move(dims)});
  }
};

struct Param : View { // (param ident type|inferred)
  explicit Param(TreeRef t) : View(std::move(t), TK_PARAM, 2) {}
  Ident ident() const { return Ident(tree_->tree(0)); }
  TreeRef type() const { return tree_->tree(1); }
  bool typeIsInferred() const { return type()->kind() == TK_INFERRED; }
  TensorType tensorType() const { return TensorType(type()); }
  static TreeRef create(const SourceRange& r, TreeRef ident, TreeRef type) {
    return Tree::make(TK_PARAM, r, {std::move(ident), std::move(type)});
  }
};

struct RangeConstraint : View { // (range_constraint ident start end)
  explicit RangeConstraint(TreeRef t) : View(std::move(t), TK_RANGE_CONSTRAINT, 3) {}
  Ident ident() const { return Ident(tree_->tree(0)); }
  TreeRef start() const { return tree_->tree(1); }
  TreeRef end() const { return tree_->tree(2); }
};

struct Let : View { // (let ident rhs)
  explicit Let(TreeRef t) : View(std::move(t), TK_LET, 2) {}
  Ident name() const { return Ident(tree_->tree(0)); }
  TreeRef rhs() const { return tree_->tree(1); }
};

struct Comprehension : View {
  // (comprehension ident (list indices) assignment rhs (list where) (option equivalent) (list reduction vars))
  explicit Comprehension(TreeRef t) : View(std::move(t), TK_COMPREHENSION, 7) {}
  Ident ident() const { return Ident(tree_->tree(0)); }
  const TreeList& indices() const { return tree_->tree(1)->trees(); }
  TreeRef assignment() const { return tree_->tree(2); }
  TreeRef rhs() const { return tree_->tree(3); }
  const TreeList& whereClauses() const { return tree_->tree(4)->trees(); }
  TreeRef equivalent() const { return tree_->tree(5); }
  const TreeList& reductionVariables() const { return tree_->tree(6)->trees(); }
};

struct Def : View { // (def ident (list params) (list returns) (list statements))
  explicit Def(TreeRef t) : View(std::move(t), TK_DEF, 4) {}
  Ident name() const { return Ident(tree_->tree(0)); }
  const TreeList& params() const { return tree_->tree(1)->trees(); }
  const TreeList& returns() const { return tree_->tree(2)->trees(); }
  const TreeList& statements() const { return tree_->tree(3)->trees(); }
};

struct Const : View { // (const number type)
  explicit Const(TreeRef t) : View(std::move(t), TK_CONST, 2) {}
  double value() const { return tree_->tree(0)->doubleValue(); }
  TreeRef type() const { return tree_->tree(1); }
};

struct Cast : View { // (cast value type)
  explicit Cast(TreeRef t) : View(std::move(t), TK_CAST, 2) {}
  TreeRef value() const { return tree_->tree(0); }
  TreeRef type() const { return tree_->tree(1); }
};

} // namespace lang
