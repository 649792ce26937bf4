// Minimal self-contained test harness (no Catch2 offline): TEST(name) { ... }
// registers a case, CHECK / REQUIRE record failures, main() runs everything.
#ifndef MINI_TEST_H
#define MINI_TEST_H

#include <cstdio>
#include <functional>
#include <string>
#include <vector>

namespace mini {
struct Case {
  std::string name;
  std::function<void()> fn;
};
inline std::vector<Case> &cases() {
  static std::vector<Case> c;
  return c;
}
inline int &failures() {
  static int f = 0;
  return f;
}
struct Registrar {
  Registrar(const char *name, std::function<void()> fn) {
    cases().push_back({name, std::move(fn)});
  }
};
struct AbortCase {};
inline int run(int argc, char **argv) {
  std::string filter = argc > 1 ? argv[1] : "";
  int ran = 0;
  for (auto &c : cases()) {
    if (!filter.empty() && c.name.find(filter) == std::string::npos)
      continue;
    const int before = failures();
    std::printf("[ RUN  ] %s\n", c.name.c_str());
    std::fflush(stdout);
    try {
      c.fn();
    } catch (const AbortCase &) {
    }
    std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL",
                c.name.c_str());
    ++ran;
  }
  std::printf("%d cases, %d failed checks\n", ran, failures());
  return failures() == 0 ? 0 : 1;
}
} // namespace mini

#define MINI_CAT2(a, b) a##b
#define MINI_CAT(a, b) MINI_CAT2(a, b)
#define TEST(name)                                                             \
  static void MINI_CAT(test_fn_, __LINE__)();                                  \
  static mini::Registrar MINI_CAT(test_reg_, __LINE__)(                        \
      name, MINI_CAT(test_fn_, __LINE__));                                     \
  static void MINI_CAT(test_fn_, __LINE__)()
#define CHECK(cond)                                                            \
  do {                                                                         \
    if (!(cond)) {                                                             \
      ++mini::failures();                                                      \
      std::printf("  CHECK failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__);  \
    }                                                                          \
  } while (0)
#define REQUIRE(cond)                                                          \
  do {                                                                         \
    if (!(cond)) {                                                             \
      ++mini::failures();                                                      \
      std::printf("  REQUIRE failed: %s (%s:%d)\n", #cond, __FILE__,           \
                  __LINE__);                                                   \
      throw mini::AbortCase();                                                 \
    }                                                                          \
  } while (0)
#define REQUIRE_OK(expr)                                                       \
  do {                                                                         \
    fusilli::ErrorObject e_ = (expr);                                          \
    if (e_.isError()) {                                                        \
      ++mini::failures();                                                      \
      std::printf("  REQUIRE_OK failed: %s -> %s: %s (%s:%d)\n", #expr,        \
                  fusilli::errorCodeName(e_.getCode()),                        \
                  e_.getMessage().c_str(), __FILE__, __LINE__);                \
      throw mini::AbortCase();                                                 \
    }                                                                          \
  } while (0)
#define REQUIRE_ASSIGN(decl, expr)                                             \
  auto MINI_CAT(eo_, __LINE__) = (expr);                                       \
  REQUIRE_OK(fusilli::ErrorObject(MINI_CAT(eo_, __LINE__)));                   \
  decl = std::move(*MINI_CAT(eo_, __LINE__));
// Expects `expr` to fail with `code` and exactly `msg`.
#define CHECK_ERROR(expr, codeExpected, msg)                                   \
  do {                                                                         \
    fusilli::ErrorObject e_ = (expr);                                          \
    if (e_.getCode() != (codeExpected) || e_.getMessage() != (msg)) {          \
      ++mini::failures();                                                      \
      std::printf("  CHECK_ERROR failed: %s\n    got  %s: %s\n    want %s: "   \
                  "%s (%s:%d)\n",                                              \
                  #expr, fusilli::errorCodeName(e_.getCode()),                 \
                  e_.getMessage().c_str(),                                     \
                  fusilli::errorCodeName(codeExpected),                        \
                  std::string(msg).c_str(), __FILE__, __LINE__);               \
    }                                                                          \
  } while (0)

#endif // MINI_TEST_H
