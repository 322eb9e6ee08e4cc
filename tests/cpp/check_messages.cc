// Message layout and exception types of the TC_CHECK family, the scenarios of the reference's
// test/test_check.cc:33-206: "Check failed [file:line]( error)(: info)", containers streamed as
// comma-separated elements, an optional exception type as last macro argument.
// Prints one line per failed expectation and returns their count.
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "tc/core/check.h"

static int failures = 0;

static std::string at(int line, const std::string& rest) {
  return std::string("Check failed [") + __FILE__ + ":" + std::to_string(line) + "]" + rest;
}

template <typename E, typename F>
static void throwsWith(F f, const std::string& expected, int line) {
  try {
    f();
    std::printf("line %d: nothing thrown\n", line);
    ++failures;
  } catch (const E& e) {
    if (expected != "*" && expected != e.what()) {
      std::printf("line %d: got \"%s\", expected \"%s\"\n", line, e.what(), expected.c_str());
      ++failures;
    }
  } catch (...) {
    std::printf("line %d: another exception type\n", line);
    ++failures;
  }
}

template <typename F>
static void quiet(F f, int line) {
  try {
    f();
  } catch (...) {
    std::printf("line %d: threw\n", line);
    ++failures;
  }
}

#define WHAT(stmt, rest) throwsWith<std::runtime_error>([&] { stmt; }, at(__LINE__, rest), __LINE__)
#define RANGE(stmt) throwsWith<std::out_of_range>([&] { stmt; }, "*", __LINE__)
#define QUIET(stmt) quiet([&] { stmt; }, __LINE__)

int main() {
  QUIET(TC_CHECK(true));
  WHAT(TC_CHECK(false), "");
  WHAT(TC_CHECK(false) << "1+1=3", ": 1+1=3");
  std::vector<int> v{1, 2, 3, 4};
  WHAT(TC_CHECK(false) << v, ": 1,2,3,4");
  WHAT(TC_CHECK(false) << "v=" << v << ";", ": v=1,2,3,4;");
  WHAT(TC_CHECK(false) << std::vector<int>{}, "");

  QUIET(TC_CHECK_EQ(1, 1));
  QUIET(TC_CHECK_EQ(std::string("aaa"), std::string("aaa")));
  WHAT(TC_CHECK_EQ(1, 2), " 1 not equal to 2");
  WHAT(TC_CHECK_EQ(1, 2) << "2+2=5", " 1 not equal to 2: 2+2=5");
  QUIET(TC_CHECK_NE(1, 2));
  WHAT(TC_CHECK_NE(1, 1), " 1 equal to 1");
  WHAT(TC_CHECK_NE(1, 1) << "2+2=5", " 1 equal to 1: 2+2=5");
  QUIET(TC_CHECK_LT(1, 2));
  WHAT(TC_CHECK_LT(1, 1), " 1 not less than 1");
  WHAT(TC_CHECK_LT(4, 1) << "4+3=8", " 4 not less than 1: 4+3=8");
  QUIET(TC_CHECK_GT(2, 1));
  WHAT(TC_CHECK_GT(1, 1), " 1 not greater than 1");
  WHAT(TC_CHECK_GT(2, 4) << "3+3=7", " 2 not greater than 4: 3+3=7");
  QUIET(TC_CHECK_LE(1, 1));
  WHAT(TC_CHECK_LE(2, 1), " 2 not less than or equal to 1");
  WHAT(TC_CHECK_LE(4, 1) << "4+5=10", " 4 not less than or equal to 1: 4+5=10");
  QUIET(TC_CHECK_GE(7, 7));
  WHAT(TC_CHECK_GE(7, 9), " 7 not greater than or equal to 9");
  WHAT(TC_CHECK_GE(2, 6) << "9+3=13", " 2 not greater than or equal to 6: 9+3=13");

  RANGE(TC_CHECK(false, std::out_of_range));
  RANGE(TC_CHECK(false, std::out_of_range) << "aa");
  QUIET(TC_CHECK(true, std::out_of_range) << "aa");
  RANGE(TC_CHECK_EQ(1, 2, std::out_of_range) << "aa");
  QUIET(TC_CHECK_EQ(1, 1, std::out_of_range) << "aa");
  RANGE(TC_CHECK_NE(1, 1, std::out_of_range));
  QUIET(TC_CHECK_NE(1, 2, std::out_of_range));
  RANGE(TC_CHECK_LT(1, 1, std::out_of_range) << "aa");
  QUIET(TC_CHECK_LT(1, 2, std::out_of_range));
  RANGE(TC_CHECK_GT(1, 1, std::out_of_range));
  QUIET(TC_CHECK_GT(2, 1, std::out_of_range) << "aa");
  RANGE(TC_CHECK_LE(2, 1, std::out_of_range));
  QUIET(TC_CHECK_LE(1, 2, std::out_of_range));
  RANGE(TC_CHECK_GE(1, 2, std::out_of_range) << "aa");
  QUIET(TC_CHECK_GE(2, 1, std::out_of_range));

  // the side of a passing check is not evaluated into the message, a failing one only once
  int calls = 0;
  auto counted = [&] { ++calls; return 5; };
  QUIET(TC_CHECK(true) << counted());
  std::printf("%d expectation(s) failed\n", failures);
  return failures;
}
