// Minimal check macros for the C++ API test programs.
#ifndef PORTDNN_AMD_TESTS_CPP_CHECK_H_
#define PORTDNN_AMD_TESTS_CPP_CHECK_H_
#include <cstdio>
#include <cstdlib>

static int g_failures = 0;
static int g_checks = 0;

#define CHECK(cond)                                                     \
  do {                                                                  \
    ++g_checks;                                                         \
    if (!(cond)) {                                                      \
      ++g_failures;                                                     \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
    }                                                                   \
  } while (0)

#define CHECK_EQ(a, b)                                                  \
  do {                                                                  \
    ++g_checks;                                                         \
    const long long va_ = static_cast<long long>(a);                    \
    const long long vb_ = static_cast<long long>(b);                    \
    if (va_ != vb_) {                                                   \
      ++g_failures;                                                     \
      std::printf("FAIL %s:%d: %s == %s (%lld vs %lld)\n", __FILE__,    \
                  __LINE__, #a, #b, va_, vb_);                          \
    }                                                                   \
  } while (0)

static inline int report(const char* name) {
  std::printf("%s: %d checks, %d failures\n", name, g_checks, g_failures);
  return g_failures == 0 ? 0 : 1;
}
#endif  // PORTDNN_AMD_TESTS_CPP_CHECK_H_
