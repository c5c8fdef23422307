// Host-side check of csrc/repeated_sum.h: the closed form against the loop it replaces, bit for bit.
// Built and run by tests/test_repeated_sum.py with the host compiler.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>

#include "../brainpylib_amd/csrc/repeated_sum.h"

template <typename F>
static F looped(F w, uint64_t n) {
  volatile F s = 0;
  for (uint64_t i = 0; i < n; ++i) s = s + w;
  return s;
}

template <typename F>
static bool same_bits(F a, F b) { return std::memcmp(&a, &b, sizeof(F)) == 0 || (a != a && b != b); }

template <typename F>
static int sweep(const char *name, uint64_t n_max, int cases) {
  std::mt19937_64 g(5);
  std::uniform_real_distribution<double> U(0, 1);
  int bad = 0;
  for (int c = 0; c < cases; ++c) {
    F w;
    switch (c % 6) {
      case 0: w = static_cast<F>(0.6); break;                                                        // the E/I net's weight
      case 1: w = static_cast<F>(std::ldexp(U(g) + 0.5, static_cast<int>(g() % 40) - 20)); break;    // any magnitude
      case 2: w = -static_cast<F>(U(g)); break;                                                      // negative
      case 3: w = static_cast<F>(1.0 + std::ldexp(1.0, -static_cast<int>(g() % 24))); break;          // exact ties
      case 4: w = static_cast<F>(std::ldexp(static_cast<double>(g() % 1000 + 1), -static_cast<int>(g() % 30))); break;
      default: w = static_cast<F>(U(g) * 1e-3); break;
    }
    const uint64_t n = (c % 7 == 0) ? g() % n_max : g() % 5000;  // long sums cross many binades and saturate
    const F want = looped<F>(w, n), got = bpl::repeated_sum<F>(w, n);
    if (!same_bits(want, got)) {
      if (bad < 10) std::printf("%s: w=%.17g n=%llu loop=%.17g closed=%.17g\n", name, static_cast<double>(w),
                                static_cast<unsigned long long>(n), static_cast<double>(want), static_cast<double>(got));
      ++bad;
    }
  }
  std::printf("%s: %d cases, %d differ\n", name, cases, bad);
  return bad;
}

int main() {
  int bad = sweep<float>("float", 40000000ull, 300) + sweep<double>("double", 10000000ull, 200);
  const float special[] = {0.f, -0.f, INFINITY, -INFINITY, NAN, 1e-45f, 3e-39f, 3.4e38f, 1.7e38f};
  for (float w : special)
    for (uint64_t n : {0ull, 1ull, 2ull, 5ull, 100ull, 20000000ull})
      if (!same_bits(looped<float>(w, n), bpl::repeated_sum<float>(w, n))) {
        std::printf("special: w=%g n=%llu\n", w, static_cast<unsigned long long>(n));
        ++bad;
      }
  return bad != 0;
}
