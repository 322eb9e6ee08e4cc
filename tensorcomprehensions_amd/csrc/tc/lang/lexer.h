// TC lexer: token kinds, source ranges and the tokenizer.
//
// Token spelling, the kind names printed in AST dumps and the "longest match, keyword beats
// identifier" rule follow the reference lexer (tc/lang/lexer.h:37-92 token table, :186-262
// matching, :206-212 '#' comments) because dumps of the tree are compared byte-for-byte with
// the reference's golden files (tc/lang/test_expected/*.expected).
#pragma once
#include <cctype>
#include <cstdlib>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace lang {

// Single-character tokens are their own kind; everything else lives above 255.
enum TokenKind : int {
  TK_EOF = 256, TK_NUMBER, TK_BOOL_VALUE, TK_MIN, TK_MAX, TK_WHERE, TK_DEF, TK_ARROW, TK_EQUIVALENT,
  TK_IDENT, TK_STRING, TK_CONST, TK_LIST, TK_OPTION, TK_APPLY, TK_COMPREHENSION, TK_TENSOR_TYPE,
  TK_RANGE_CONSTRAINT, TK_PARAM, TK_INFERRED, TK_ACCESS, TK_BUILT_IN, TK_PLUS_EQ, TK_TIMES_EQ,
  TK_MIN_EQ, TK_MAX_EQ, TK_PLUS_EQ_B, TK_TIMES_EQ_B, TK_MIN_EQ_B, TK_MAX_EQ_B, TK_BOOL, TK_UINT8,
  TK_UINT16, TK_UINT32, TK_UINT64, TK_INT8, TK_INT16, TK_INT32, TK_INT64, TK_FLOAT16, TK_FLOAT32,
  TK_FLOAT64, TK_FLOAT, TK_DOUBLE, TK_CAST, TK_IN, TK_GE, TK_LE, TK_EQ, TK_NE, TK_AND, TK_OR,
  TK_LET, TK_EXISTS, TK_DEF_END_
};

struct TokenSpec {
  int kind;
  const char* name;     // printed in dumps and error messages
  const char* spelling; // "" when the lexer never produces it from text
};

inline const std::vector<TokenSpec>& tokenTable() {
  static const std::vector<TokenSpec> t = {
      {TK_EOF, "eof", ""}, {TK_NUMBER, "number", ""}, {TK_BOOL_VALUE, "bool_value", ""},
      {TK_MIN, "min", "min"}, {TK_MAX, "max", "max"}, {TK_WHERE, "where", "where"},
      {TK_DEF, "def", "def"}, {TK_ARROW, "arrow", "->"}, {TK_EQUIVALENT, "equivalent", "<=>"},
      {TK_IDENT, "ident", ""}, {TK_STRING, "string", ""}, {TK_CONST, "const", ""},
      {TK_LIST, "list", ""}, {TK_OPTION, "option", ""}, {TK_APPLY, "apply", ""},
      {TK_COMPREHENSION, "comprehension", ""}, {TK_TENSOR_TYPE, "tensor_type", ""},
      {TK_RANGE_CONSTRAINT, "range_constraint", ""}, {TK_PARAM, "param", ""},
      {TK_INFERRED, "inferred", ""}, {TK_ACCESS, "access", ""}, {TK_BUILT_IN, "built-in", ""},
      {TK_PLUS_EQ, "plus_eq", "+="}, {TK_TIMES_EQ, "times_eq", "*="}, {TK_MIN_EQ, "min_eq", "min="},
      {TK_MAX_EQ, "max_eq", "max="}, {TK_PLUS_EQ_B, "plus_eq_b", "+=!"},
      {TK_TIMES_EQ_B, "times_eq_b", "*=!"}, {TK_MIN_EQ_B, "min_eq_b", "min=!"},
      {TK_MAX_EQ_B, "max_eq_b", "max=!"}, {TK_BOOL, "bool", "bool"}, {TK_UINT8, "uint8", "uint8"},
      {TK_UINT16, "uint16", "uint16"}, {TK_UINT32, "uint32", "uint32"}, {TK_UINT64, "uint64", "uint64"},
      {TK_INT8, "int8", "int8"}, {TK_INT16, "int16", "int16"}, {TK_INT32, "int32", "int32"},
      {TK_INT64, "int64", "int64"}, {TK_FLOAT16, "float16", "float16"},
      {TK_FLOAT32, "float32", "float32"}, {TK_FLOAT64, "float64", "float64"},
      {TK_FLOAT, "float", "float"}, {TK_DOUBLE, "double", "double"}, {TK_CAST, "cast", ""},
      {TK_IN, "in", "in"}, {TK_GE, "ge", ">="}, {TK_LE, "le", "<="}, {TK_EQ, "eq", "=="},
      {TK_NE, "neq", "!="}, {TK_AND, "and", "&&"}, {TK_OR, "or", "||"}, {TK_LET, "let", ""},
      {TK_EXISTS, "exists", "exists"}};
  return t;
}

inline const char* singleCharTokens() {
  return "+-*/()[]?:,={}><!%";
}

inline std::string kindToString(int kind) {
  if (kind < 256) {
    return std::string(1, static_cast<char>(kind));
  }
  for (const auto& s : tokenTable()) {
    if (s.kind == kind) {
      return s.name;
    }
  }
  throw std::runtime_error("unknown token kind " + std::to_string(kind));
}

// Text the lexer matches for a kind ("+=" for TK_PLUS_EQ); throws for AST-only kinds.
inline std::string kindToToken(int kind) {
  if (kind < 256) {
    return std::string(1, static_cast<char>(kind));
  }
  for (const auto& s : tokenTable()) {
    if (s.kind == kind && s.spelling[0] != '\0') {
      return s.spelling;
    }
  }
  throw std::runtime_error("token kind has no spelling: " + std::to_string(kind));
}

inline bool isScalarTypeKind(int kind) {
  return kind >= TK_BOOL && kind <= TK_DOUBLE;
}

// A half-open character range [start, end) of a shared source string.
class SourceRange {
 public:
  SourceRange(std::shared_ptr<std::string> file, size_t start, size_t end)
      : file_(std::move(file)), start_(start), end_(end) {}
  const std::string& file() const { return *file_; }
  const std::shared_ptr<std::string>& file_ptr() const { return file_; }
  size_t start() const { return start_; }
  size_t end() const { return end_; }
  size_t size() const { return end_ - start_; }
  std::string text() const { return file_->substr(start_, size()); }

  // Prints the source up to and including the line holding the range, a row of '~' under the
  // range, then the rest of the source (layout fixed by tc/lang/test_expected/lexer.expected).
  void highlight(std::ostream& out) const {
    const std::string& s = *file_;
    size_t lineBegin = start_, lineEnd = start_;
    while (lineBegin > 0 && s[lineBegin - 1] != '\n') {
      --lineBegin;
    }
    while (lineEnd < s.size() && s[lineEnd] != '\n') {
      ++lineEnd;
    }
    out << s.substr(0, lineEnd) << "\n" << std::string(start_ - lineBegin, ' ');
    size_t shown = std::min(size(), lineEnd - start_);
    out << std::string(shown, '~') << (shown < size() ? "...  <--- HERE" : " <--- HERE");
    out << s.substr(lineEnd);
    if (!s.empty() && s.back() != '\n') {
      out << "\n";
    }
  }

 private:
  std::shared_ptr<std::string> file_;
  size_t start_, end_;
};

// Exception carrying a message followed by the highlighted source location.
class ErrorReport : public std::exception {
 public:
  explicit ErrorReport(const SourceRange& r) : range_(r) {}
  ErrorReport(const ErrorReport& o) : range_(o.range_), what_() { ss_ << o.ss_.str(); }
  template <typename T>
  ErrorReport& operator<<(const T& v) {
    ss_ << v;
    return *this;
  }
  const char* what() const noexcept override {
    std::stringstream out;
    out << ss_.str() << ":\n";
    range_.highlight(out);
    what_ = out.str();
    return what_.c_str();
  }
  std::string message() const { return ss_.str(); }

 private:
  SourceRange range_;
  std::stringstream ss_;
  mutable std::string what_;
};

struct Token {
  int kind;
  SourceRange range;
  std::string text() const { return range.text(); }
  double doubleValue() const { return std::strtod(text().c_str(), nullptr); }
};

class Lexer {
 public:
  explicit Lexer(const std::string& src)
      : file_(std::make_shared<std::string>(src)), cur_{TK_EOF, SourceRange(file_, 0, 0)} {
    next();
  }
  Token& cur() { return cur_; }
  Token next() {
    Token prev = cur_;
    if (hasAhead_) {
      cur_ = ahead_[0];
      hasAhead_ = false;
      ahead_.clear();
    } else {
      cur_ = scan();
    }
    return prev;
  }
  Token lookahead() {
    if (!hasAhead_) {
      ahead_.push_back(scan());
      hasAhead_ = true;
    }
    return ahead_[0];
  }
  bool nextIf(int kind) {
    if (cur_.kind != kind) {
      return false;
    }
    next();
    return true;
  }
  Token expect(int kind) {
    if (cur_.kind != kind) {
      reportError(kindToString(kind));
    }
    return next();
  }
  [[noreturn]] void reportError(const std::string& what, const Token& t) {
    ErrorReport e(t.range);
    e << "expected " << what << " but found '" << kindToString(t.kind) << "' here";
    throw e;
  }
  [[noreturn]] void reportError(const std::string& what) { reportError(what, cur_); }
  const std::shared_ptr<std::string>& file() const { return file_; }

 private:
  static bool identChar(size_t i, char c) {
    return std::isalpha(static_cast<unsigned char>(c)) || c == '_' ||
        (i > 0 && std::isdigit(static_cast<unsigned char>(c)));
  }
  Token scan() {
    const std::string& s = *file_;
    // whitespace and '#' comments
    for (;;) {
      while (pos_ < s.size() && std::isspace(static_cast<unsigned char>(s[pos_]))) {
        ++pos_;
      }
      if (pos_ < s.size() && s[pos_] == '#') {
        while (pos_ < s.size() && s[pos_] != '\n') {
          ++pos_;
        }
        continue;
      }
      break;
    }
    size_t start = pos_;
    if (pos_ == s.size()) {
      return Token{TK_EOF, SourceRange(file_, start, start)};
    }
    // numbers: whatever strtod accepts, minus a leading sign (so "1+3" stays three tokens)
    if (s[start] != '-' && s[start] != '+') {
      const char* b = s.c_str() + start;
      char* e = nullptr;
      std::strtod(b, &e);
      if (e > b) {
        pos_ = start + static_cast<size_t>(e - b);
        return Token{TK_NUMBER, SourceRange(file_, start, pos_)};
      }
    }
    // longest identifier
    size_t idLen = 0;
    while (start + idLen < s.size() && identChar(idLen, s[start + idLen])) {
      ++idLen;
    }
    // longest spelled token (keywords and operators); on a tie the token wins over the identifier
    size_t tokLen = 0;
    int tokKind = 0;
    for (const auto& spec : tokenTable()) {
      size_t n = std::char_traits<char>::length(spec.spelling);
      if (n > tokLen && s.compare(start, n, spec.spelling) == 0) {
        tokLen = n;
        tokKind = spec.kind;
      }
    }
    if (tokLen == 0) {
      for (const char* c = singleCharTokens(); *c; ++c) {
        if (*c == s[start]) {
          tokLen = 1;
          tokKind = *c;
        }
      }
    }
    if (idLen > tokLen) {
      pos_ = start + idLen;
      return Token{TK_IDENT, SourceRange(file_, start, pos_)};
    }
    if (tokLen > 0) {
      pos_ = start + tokLen;
      return Token{tokKind, SourceRange(file_, start, pos_)};
    }
    Token bad{static_cast<unsigned char>(s[start]), SourceRange(file_, start, start + 1)};
    ErrorReport e(bad.range);
    e << "expected a valid token but found '" << s[start] << "' here";
    throw e;
  }

  std::shared_ptr<std::string> file_;
  size_t pos_ = 0;
  Token cur_;
  std::vector<Token> ahead_;
  bool hasAhead_ = false;
};

} // namespace lang
