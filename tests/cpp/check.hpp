// Minimal test harness for the C++ host-surface tests: each TEST registers itself,
// main() runs them all (or those whose name contains argv[1]) and exits non-zero
// on the first failed CHECK.  Every test body runs on a fresh thread, because the
// runtime's device contexts are thread-local (the reference isolates its tests
// the same way, cuda-async/tests/cuda_graph.rs:18-20).
#pragma once
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

struct TestCase {
  const char* name;
  std::function<void()> fn;
};
inline std::vector<TestCase>& test_registry() {
  static std::vector<TestCase> r;
  return r;
}
struct TestRegistrar {
  TestRegistrar(const char* name, std::function<void()> fn) { test_registry().push_back({name, std::move(fn)}); }
};
#define TEST(name)                                          \
  static void test_##name();                                \
  static TestRegistrar registrar_##name(#name, test_##name); \
  static void test_##name()

struct CheckFailure : std::runtime_error {
  using std::runtime_error::runtime_error;
};
#define CHECK(cond)                                                                                       \
  do {                                                                                                    \
    if (!(cond)) throw CheckFailure(std::string(__FILE__) + ":" + std::to_string(__LINE__) + ": CHECK(" #cond ") failed"); \
  } while (0)
#define CHECK_MSG(cond, msg)                                                                               \
  do {                                                                                                     \
    if (!(cond)) throw CheckFailure(std::string(__FILE__) + ":" + std::to_string(__LINE__) + ": CHECK(" #cond ") failed: " + (msg)); \
  } while (0)
#define CHECK_THROWS(expr, needle)                                                        \
  do {                                                                                    \
    bool threw = false;                                                                   \
    try {                                                                                 \
      (void)(expr);                                                                       \
    } catch (const CheckFailure&) {                                                       \
      throw;                                                                              \
    } catch (const std::exception& e) {                                                   \
      threw = true;                                                                       \
      CHECK_MSG(std::string(e.what()).find(needle) != std::string::npos, e.what());       \
    }                                                                                     \
    CHECK_MSG(threw, "expected an exception containing: " needle);                        \
  } while (0)

inline int run_all_tests(int argc, char** argv) {
  const char* filter = argc > 1 ? argv[1] : "";
  int ran = 0;
  for (auto& t : test_registry()) {
    if (*filter && !strstr(t.name, filter)) continue;
    std::string failure;
    printf("RUN  %s\n", t.name);
    fflush(stdout);
    std::thread th([&] {
      try {
        t.fn();
      } catch (const std::exception& e) {
        failure = e.what();
      }
    });
    th.join();
    if (!failure.empty()) {
      printf("FAIL %s: %s\n", t.name, failure.c_str());
      return 1;
    }
    printf("PASS %s\n", t.name);
    ++ran;
  }
  printf("ALL %d TESTS PASSED\n", ran);
  return 0;
}
