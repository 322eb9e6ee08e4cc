// TC_CHECK family: condition checks that throw with a "Check failed [file:line] ..." message.
// Usage and message layout mirror the reference's macros (tc/core/check.h:35-120):
//   TC_CHECK_EQ(x, 42) << "x is not the answer";
//   TC_CHECK_LT(i, n, std::out_of_range) << "...";
// The exception is thrown from the temporary's destructor, at the end of the full expression.
#pragma once
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>

namespace tc {
namespace detail {

// containers with begin()/end() other than strings
template <typename T, typename = void>
struct IsContainer : std::false_type {};
template <typename T>
struct IsContainer<T, decltype(void(std::declval<const T&>().begin()), void(std::declval<const T&>().end()))>
    : std::integral_constant<bool, !std::is_convertible<T, std::string>::value> {};

template <typename E>
class Checker {
 public:
  Checker(bool ok, const char* file, int line, std::string what)
      : ok_(ok), file_(file), line_(line), what_(std::move(what)) {}
  Checker(Checker&& o) : ok_(o.ok_), file_(o.file_), line_(o.line_), what_(o.what_) {
    info_ << o.info_.str();
    o.ok_ = true;
  }
  ~Checker() noexcept(false) {
    if (ok_) {
      return;
    }
    // "Check failed [file:line]( error)(: info)", the layout test/test_check.cc:33-166 pins
    std::stringstream ss;
    ss << "Check failed [" << file_ << ':' << line_ << ']';
    if (!what_.empty()) {
      ss << ' ' << what_;
    }
    if (!info_.str().empty()) {
      ss << ": " << info_.str();
    }
    throw E(ss.str());
  }
  template <typename T>
  typename std::enable_if<!IsContainer<T>::value, Checker&>::type operator<<(const T& v) {
    if (!ok_) {
      info_ << v;
    }
    return *this;
  }
  // a standard container prints its elements separated by commas
  template <typename C>
  typename std::enable_if<IsContainer<C>::value, Checker&>::type operator<<(const C& c) {
    if (!ok_) {
      bool first = true;
      for (const auto& x : c) {
        info_ << (first ? "" : ",") << x;
        first = false;
      }
    }
    return *this;
  }

 private:
  bool ok_;
  const char* file_;
  int line_;
  std::string what_;
  std::stringstream info_;
};

template <typename E, typename X, typename Y>
Checker<E> compare(bool ok, const X& x, const Y& y, const char* rel, const char* file, int line) {
  std::stringstream ss;
  if (!ok) {
    ss << x << " " << rel << " " << y;
  }
  return Checker<E>(ok, file, line, ss.str());
}

} // namespace detail
} // namespace tc

#define TC_CHECK_PICK3_(_1, _2, _3, NAME, ...) NAME
#define TC_CHECK_PICK2_(_1, _2, NAME, ...) NAME
#define TC_CHECK_1_(c) ::tc::detail::Checker<std::runtime_error>(static_cast<bool>(c), __FILE__, __LINE__, "")
#define TC_CHECK_2_(c, E) ::tc::detail::Checker<E>(static_cast<bool>(c), __FILE__, __LINE__, "")
#define TC_CHECK(...) TC_CHECK_PICK2_(__VA_ARGS__, TC_CHECK_2_, TC_CHECK_1_)(__VA_ARGS__)

#define TC_CMP_2_(op, rel, x, y) \
  ::tc::detail::compare<std::runtime_error>((x)op(y), (x), (y), rel, __FILE__, __LINE__)
#define TC_CMP_3_(op, rel, x, y, E) ::tc::detail::compare<E>((x)op(y), (x), (y), rel, __FILE__, __LINE__)
#define TC_CHECK_EQ_2_(x, y) TC_CMP_2_(==, "not equal to", x, y)
#define TC_CHECK_EQ_3_(x, y, E) TC_CMP_3_(==, "not equal to", x, y, E)
#define TC_CHECK_NE_2_(x, y) TC_CMP_2_(!=, "equal to", x, y)
#define TC_CHECK_NE_3_(x, y, E) TC_CMP_3_(!=, "equal to", x, y, E)
#define TC_CHECK_LT_2_(x, y) TC_CMP_2_(<, "not less than", x, y)
#define TC_CHECK_LT_3_(x, y, E) TC_CMP_3_(<, "not less than", x, y, E)
#define TC_CHECK_GT_2_(x, y) TC_CMP_2_(>, "not greater than", x, y)
#define TC_CHECK_GT_3_(x, y, E) TC_CMP_3_(>, "not greater than", x, y, E)
#define TC_CHECK_LE_2_(x, y) TC_CMP_2_(<=, "not less than or equal to", x, y)
#define TC_CHECK_LE_3_(x, y, E) TC_CMP_3_(<=, "not less than or equal to", x, y, E)
#define TC_CHECK_GE_2_(x, y) TC_CMP_2_(>=, "not greater than or equal to", x, y)
#define TC_CHECK_GE_3_(x, y, E) TC_CMP_3_(>=, "not greater than or equal to", x, y, E)
#define TC_CHECK_EQ(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_EQ_3_, TC_CHECK_EQ_2_)(__VA_ARGS__)
#define TC_CHECK_NE(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_NE_3_, TC_CHECK_NE_2_)(__VA_ARGS__)
#define TC_CHECK_LT(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_LT_3_, TC_CHECK_LT_2_)(__VA_ARGS__)
#define TC_CHECK_GT(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_GT_3_, TC_CHECK_GT_2_)(__VA_ARGS__)
#define TC_CHECK_LE(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_LE_3_, TC_CHECK_LE_2_)(__VA_ARGS__)
#define TC_CHECK_GE(...) TC_CHECK_PICK3_(__VA_ARGS__, TC_CHECK_GE_3_, TC_CHECK_GE_2_)(__VA_ARGS__)
