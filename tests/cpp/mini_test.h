// A few dozen lines of test plumbing in the shape of the GoogleTest subset the
// reference's tests use (TEST, EXPECT_*, ASSERT_*), so the cases below read like
// src/llm/layers/*_test.cc.  Tests whose suite name ends in "Cpu" need no GPU.
#pragma once

#include <cmath>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace mini_test {

struct Case {
  std::string suite, name;
  std::function<void()> body;
};

inline std::vector<Case>& Registry() {
  static std::vector<Case> cases;
  return cases;
}
inline int& Failures() {
  static int failures = 0;
  return failures;
}
struct Registrar {
  Registrar(const char* suite, const char* name, std::function<void()> body) {
    Registry().push_back({suite, name, std::move(body)});
  }
};

// Collects the streamed message of a failed check and prints it on destruction.
class Failure {
 public:
  Failure(const char* file, int line, const std::string& what) {
    ++Failures();
    text_ << file << ":" << line << ": " << what;
  }
  ~Failure() { std::cout << text_.str() << std::endl; }
  template <class T>
  Failure& operator<<(const T& value) {
    text_ << " " << value;
    return *this;
  }

 private:
  std::ostringstream text_;
};

struct Voidify {
  void operator&(const Failure&) {}
};

template <class A, class B>
std::string Describe(const char* op, const char* a_text, const char* b_text, const A& a,
                     const B& b) {
  std::ostringstream out;
  out << "expected " << a_text << " " << op << " " << b_text;
  if constexpr (requires(std::ostream& o) { o << a; o << b; })
    out << " (" << a << " vs " << b << ")";
  return out.str();
}

}  // namespace mini_test

#define TEST(suite, name)                                                                  \
  static void suite##_##name##_body();                                                     \
  static ::mini_test::Registrar suite##_##name##_registrar(#suite, #name,                  \
                                                           suite##_##name##_body);         \
  static void suite##_##name##_body()

#define MINI_CHECK_(condition, what, on_failure)                                           \
  if (condition)                                                                           \
    ;                                                                                      \
  else                                                                                     \
    on_failure ::mini_test::Voidify() & ::mini_test::Failure(__FILE__, __LINE__, what)

#define EXPECT_TRUE(c) MINI_CHECK_((c), "expected true: " #c, )
#define EXPECT_FALSE(c) MINI_CHECK_(!(c), "expected false: " #c, )
#define ASSERT_TRUE(c) MINI_CHECK_((c), "expected true: " #c, return)
#define ASSERT_FALSE(c) MINI_CHECK_(!(c), "expected false: " #c, return)
#define MINI_COMPARE_(a, b, op, on_failure) \
  MINI_CHECK_((a)op(b), ::mini_test::Describe(#op, #a, #b, (a), (b)), on_failure)
#define EXPECT_EQ(a, b) MINI_COMPARE_(a, b, ==, )
#define EXPECT_NE(a, b) MINI_COMPARE_(a, b, !=, )
#define EXPECT_GT(a, b) MINI_COMPARE_(a, b, >, )
#define EXPECT_LE(a, b) MINI_COMPARE_(a, b, <=, )
#define ASSERT_EQ(a, b) MINI_COMPARE_(a, b, ==, return)
#define EXPECT_NEAR(a, b, tolerance)                                                       \
  MINI_CHECK_(std::fabs(double(a) - double(b)) <= double(tolerance),                       \
              ::mini_test::Describe("~=", #a, #b, (a), (b)), )
