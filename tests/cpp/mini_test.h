// A few lines of test harness (no gtest in this build): TEST(suite, name) registers
// a function, main() runs them all, ASSERT_* print and fail the current test.
#pragma once
#include <cstdio>
#include <functional>
#include <string>
#include <vector>

namespace mini {
struct Case {
  std::string name;
  std::function<void(bool&)> fn;
};
inline std::vector<Case>& cases() {
  static std::vector<Case> c;
  return c;
}
struct Registrar {
  Registrar(const char* suite, const char* name, std::function<void(bool&)> fn) {
    cases().push_back({std::string(suite) + "." + name, std::move(fn)});
  }
};
inline int run_all() {
  int failed = 0;
  for (auto& c : cases()) {
    bool ok = true;
    printf("[ RUN      ] %s\n", c.name.c_str());
    fflush(stdout);
    c.fn(ok);
    printf("[ %s ] %s\n", ok ? "      OK" : "  FAILED", c.name.c_str());
    fflush(stdout);
    failed += ok ? 0 : 1;
  }
  printf("%zu tests, %d failed\n", cases().size(), failed);
  return failed == 0 ? 0 : 1;
}
}  // namespace mini

#define TEST(suite, name)                                                    \
  static void suite##_##name##_body(bool& mini_ok);                          \
  static mini::Registrar suite##_##name##_reg(#suite, #name, suite##_##name##_body); \
  static void suite##_##name##_body(bool& mini_ok)

#define ASSERT_EQ(a, b)                                                              \
  do {                                                                               \
    const auto mini_a = (a);                                                         \
    const auto mini_b = (b);                                                         \
    if (!(mini_a == mini_b)) {                                                       \
      printf("%s:%d: ASSERT_EQ(%s, %s) failed: %lld vs %lld\n", __FILE__, __LINE__, #a, #b, \
             static_cast<long long>(mini_a), static_cast<long long>(mini_b));        \
      mini_ok = false;                                                               \
      return;                                                                        \
    }                                                                                \
  } while (0)

#define ASSERT_TRUE(c)                                                   \
  do {                                                                   \
    if (!(c)) {                                                          \
      printf("%s:%d: ASSERT_TRUE(%s) failed\n", __FILE__, __LINE__, #c); \
      mini_ok = false;                                                   \
      return;                                                            \
    }                                                                    \
  } while (0)

#define HIP_ERROR_ASSERT(expr) ASSERT_EQ((expr), hipSuccess)
