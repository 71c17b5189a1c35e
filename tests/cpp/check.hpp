// Minimal test scaffolding for the C++ API tests: named cases, CHECK macros, the
// comparators of the reference's test utilities (cpp/tests/test_utils.h:17-45).
#pragma once

#include <cmath>
#include <cstdio>
#include <functional>
#include <string>
#include <vector>

namespace t {
struct Case {
  std::string name;
  std::function<void()> fn;
};
inline std::vector<Case>& cases()
{
  static std::vector<Case> c;
  return c;
}
inline int& failures()
{
  static int f = 0;
  return f;
}
struct Register {
  Register(const char* n, std::function<void()> f) { cases().push_back({n, std::move(f)}); }
};
inline int run_all()
{
  int bad_cases = 0;
  for (auto& c : cases()) {
    const int before = failures();
    std::printf("[ RUN  ] %s\n", c.name.c_str());
    std::fflush(stdout);
    try {
      c.fn();
    } catch (const std::exception& e) {
      std::printf("  unexpected exception: %s\n", e.what());
      ++failures();
    }
    const bool ok = failures() == before;
    bad_cases += !ok;
    std::printf("[ %s ] %s\n", ok ? " OK " : "FAIL", c.name.c_str());
  }
  std::printf("%zu cases, %d failed\n", cases().size(), bad_cases);
  return bad_cases == 0 ? 0 : 1;
}

// pass if the absolute OR the relative difference is within eps
template <typename T>
struct CompareApprox {
  explicit CompareApprox(T eps_) : eps(eps_) {}
  bool operator()(const T& a, const T& b) const
  {
    const T diff = std::abs(a - b);
    const T m    = std::max(std::abs(a), std::abs(b));
    const T ratio = diff > eps ? diff / m : diff;
    return ratio <= eps;
  }
  T eps;
};
}  // namespace t

#define TEST_CASE(name)                                   \
  static void name();                                     \
  static t::Register reg_##name(#name, name);             \
  static void name()

#define CHECK(cond)                                                            \
  do {                                                                         \
    if (!(cond)) {                                                             \
      std::printf("  %s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond);   \
      ++t::failures();                                                         \
    }                                                                          \
  } while (0)

#define CHECK_THROWS_AS(expr, type)                                                     \
  do {                                                                                  \
    bool caught_ = false;                                                               \
    try {                                                                               \
      expr;                                                                             \
    } catch (const type&) {                                                             \
      caught_ = true;                                                                   \
    } catch (...) {                                                                     \
    }                                                                                   \
    if (!caught_) {                                                                     \
      std::printf("  %s:%d: expected %s from: %s\n", __FILE__, __LINE__, #type, #expr); \
      ++t::failures();                                                                  \
    }                                                                                   \
  } while (0)
