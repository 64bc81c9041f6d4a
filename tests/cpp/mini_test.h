// A few lines of test plumbing: TEST(suite, name, needs_gpu) registers a function; CHECK*
// record failures; main() in the test file runs the selected subset and prints one line per
// test ("ok" / "FAILED") plus a summary, exiting non-zero on any failure.
#pragma once
#include <cmath>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace mini {

struct Case {
  std::string name;
  bool needs_gpu;
  std::function<void()> body;
};
inline std::vector<Case>& cases() {
  static std::vector<Case> all;
  return all;
}
inline int& failures_in_current() {
  static int n = 0;
  return n;
}
struct Registrar {
  Registrar(const char* suite, const char* name, bool gpu, std::function<void()> body) {
    cases().push_back({std::string(suite) + "." + name, gpu, std::move(body)});
  }
};
inline void fail(const char* file, int line, const std::string& what) {
  ++failures_in_current();
  std::cout << "    " << file << ":" << line << ": " << what << std::endl;
}

// mode: "cpu" (tests that need no device), "gpu" (tests that need one) or "all".
inline int run(const std::string& mode, const std::string& filter) {
  int ran = 0, failed = 0;
  for (auto& c : cases()) {
    if (mode == "cpu" && c.needs_gpu) continue;
    if (mode == "gpu" && !c.needs_gpu) continue;
    if (!filter.empty() && c.name.find(filter) == std::string::npos) continue;
    failures_in_current() = 0;
    std::cout << "[ RUN  ] " << c.name << std::endl;
    try {
      c.body();
    } catch (const std::exception& e) {
      fail("(exception)", 0, e.what());
    } catch (const char* e) {
      fail("(exception)", 0, e);
    } catch (...) {
      fail("(exception)", 0, "unknown exception");
    }
    ++ran;
    if (failures_in_current()) {
      ++failed;
      std::cout << "[FAILED] " << c.name << std::endl;
    } else {
      std::cout << "[  ok  ] " << c.name << std::endl;
    }
  }
  std::cout << "SUMMARY ran=" << ran << " failed=" << failed << std::endl;
  return failed == 0 && ran > 0 ? 0 : 1;
}

}  // namespace mini

#define TEST(suite, name, gpu)                                                     \
  static void suite##_##name();                                                    \
  static mini::Registrar reg_##suite##_##name(#suite, #name, gpu, suite##_##name); \
  static void suite##_##name()

#define CHECK(cond)                                                  \
  do {                                                               \
    if (!(cond)) mini::fail(__FILE__, __LINE__, "CHECK(" #cond ")"); \
  } while (0)
#define CHECK_EQ(a, b)                                                              \
  do {                                                                              \
    auto va = (a);                                                                  \
    auto vb = (b);                                                                  \
    if (!(va == vb)) {                                                              \
      std::ostringstream os;                                                        \
      os << "CHECK_EQ(" #a ", " #b "): " << va << " vs " << vb;                     \
      mini::fail(__FILE__, __LINE__, os.str());                                     \
    }                                                                               \
  } while (0)
#define CHECK_NEAR(a, b, tol)                                                       \
  do {                                                                              \
    double va = (a), vb = (b);                                                      \
    if (!(std::fabs(va - vb) <= (tol))) {                                           \
      std::ostringstream os;                                                        \
      os << "CHECK_NEAR(" #a ", " #b "): " << va << " vs " << vb;                   \
      mini::fail(__FILE__, __LINE__, os.str());                                     \
    }                                                                               \
  } while (0)
#define CHECK_THROWS(expr)                                                          \
  do {                                                                              \
    bool threw = false;                                                             \
    try {                                                                           \
      (void)(expr);                                                                 \
    } catch (...) {                                                                 \
      threw = true;                                                                 \
    }                                                                               \
    if (!threw) mini::fail(__FILE__, __LINE__, "CHECK_THROWS(" #expr ")");          \
  } while (0)
