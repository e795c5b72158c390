// Minimal stand-in for the gtest macros, used ONLY by the fixture generator
// (tests/golden/make_fixtures.py). Instead of judging results it records the
// expected vectors a test compares against, next to the graph the test built.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

namespace tvxcap {
struct Sink {
  template <typename T>
  const Sink& operator<<(const T&) const { return *this; }
};
struct Reg {
  Reg(const char* suite, const char* name, void (*body)());
};
void RecordGolden(const std::vector<double>& golden, double tol, const char* how);

template <typename T>
std::vector<double> ToDouble(const std::vector<T>& v) {
  std::vector<double> d;
  d.reserve(v.size());
  for (const auto& x : v) d.push_back(static_cast<double>(static_cast<float>(x)));
  return d;
}
template <typename T>
Sink RecordEq(const std::vector<T>& golden, const std::vector<T>&) {
  RecordGolden(ToDouble(golden), 0.0, "eq");
  return Sink();
}
// shapes (EXPECT_EQ(tensor->GetShape(), expected_shape)) are not output vectors
inline Sink RecordEq(const std::vector<uint32_t>&, const std::vector<uint32_t>&) { return Sink(); }
template <typename A, typename B>
Sink RecordEq(const A&, const B&) { return Sink(); }
Sink Check(bool ok, const char* expr);
// EXPECT_NEAR(golden[i], output[i], tol) in a loop over the output: the scalars are gathered and
// become one case when the test body ends, if there is one of them per output element.
Sink RecordNear(double golden, double tol);
// memcmp(output, expected, bytes) == 0 inside EXPECT_TRUE: `expected` becomes the golden vector
int RecordMem(const void* output, const void* expected, size_t bytes);
}  // namespace tvxcap

namespace testing {
struct AssertionResult {
  bool ok;
  operator bool() const { return ok; }
};
inline AssertionResult AssertionSuccess() { return AssertionResult{true}; }
inline AssertionResult AssertionFailure() { return AssertionResult{false}; }
template <typename T>
struct Matcher {
  Matcher() {}
};
inline Matcher<float> FloatNear(float, float) { return Matcher<float>(); }
}  // namespace testing

#define TEST(suite, name)                                              \
  static void suite##_##name##_body();                                 \
  static ::tvxcap::Reg suite##_##name##_reg(#suite, #name,             \
                                            &suite##_##name##_body);   \
  static void suite##_##name##_body()
#define EXPECT_TRUE(x) ::tvxcap::Check(static_cast<bool>(x), #x)
#define ASSERT_TRUE(x) ::tvxcap::Check(static_cast<bool>(x), #x)
#define EXPECT_EQ(a, b) ::tvxcap::RecordEq((a), (b))
#define EXPECT_NEAR(a, b, t) ::tvxcap::RecordNear(static_cast<double>(a), static_cast<double>(static_cast<float>(t)))
#define memcmp(a, b, n) ::tvxcap::RecordMem((a), (b), (n))
#define GTEST_SKIP() return
