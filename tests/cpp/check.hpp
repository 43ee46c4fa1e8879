#pragma once
// Minimal check counter shared by the C++ gate executables: each binary prints
// "<suite>: N checks, F failures" and exits with F (capped at 255).
#include <cstdio>
#include <stdexcept>

struct Checks {
  int checks = 0, fails = 0;
  void expect(bool ok, const char* what) {
    ++checks;
    if (!ok) {
      ++fails;
      std::printf("FAIL %s\n", what);
    }
  }
  template <class F>
  void throws_invalid(F&& f, const char* what) {
    bool got = false;
    try {
      f();
    } catch (const std::invalid_argument&) {
      got = true;
    } catch (...) {
    }
    ++checks;
    if (!got) {
      ++fails;
      std::printf("FAIL no std::invalid_argument: %s\n", what);
    }
  }
  int finish(const char* suite) const {
    std::printf("%s: %d checks, %d failures\n", suite, checks, fails);
    return fails > 255 ? 255 : fails;
  }
};
