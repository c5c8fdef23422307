// The value a loop `s = 0; repeat n times: s = s + w` leaves in s when every addition rounds to
// nearest-even in the precision of F, computed without running the loop.
//
// The reference's scatter loops add a homogeneous weight once per delivered synapse, in place, in
// the precision of the output (brainpylib/_src/event_ops/event_csr_matvec.py:313-331,
// lib/cpu_event_sum.cc:5-24).  All addends being equal, the order in which they arrive does not
// matter: the result is a function of (w, n) alone, and it is NOT n * w rounded once (with w = 0.6
// the two differ by more than 1e-5 relative from a few thousand addends on, because inside one
// binade every step makes the same rounding error).  Kernels that count synapses in integers get
// the reference's bits from the count with this function.
//
// How: while the running sum s stays inside one binade [2^e, 2^(e+1)) it is a multiple of the
// binade's spacing u, and s + w rounds to s + d with a step d (a multiple of u) that does not
// depend on s, except in the tie case (w mod u == u/2), where ties-to-even makes the quotient s/u
// even after one step and the step constant from then on.  So three real additions that stay in
// one binade establish d, and the rest of the binade is crossed at once: s + j * d is exact.
// About six additions and one division per binade, at most a few hundred operations in all.
#pragma once

#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#define BPL_HOST_DEVICE __host__ __device__
#else
#define BPL_HOST_DEVICE
#endif

namespace bpl {

template <typename F>
struct FloatFormat;
template <>
struct FloatFormat<float> {
  using Bits = uint32_t;
  static constexpr int kMantissa = 23;
  static constexpr uint32_t kExpMask = 0xffu;
};
template <>
struct FloatFormat<double> {
  using Bits = uint64_t;
  static constexpr int kMantissa = 52;
  static constexpr uint32_t kExpMask = 0x7ffu;
};

template <typename F>
BPL_HOST_DEVICE inline uint32_t biased_exponent(F v) {
  typename FloatFormat<F>::Bits b;
  memcpy(&b, &v, sizeof(F));
  return static_cast<uint32_t>(b >> FloatFormat<F>::kMantissa) & FloatFormat<F>::kExpMask;
}

// 2^(e - bias) for a biased exponent 0 < e < kExpMask (e = 1: the smallest normal number, the top of the
// subnormal range, in which sums are exact and the step is w itself)
template <typename F>
BPL_HOST_DEVICE inline F power_of_two(uint32_t biased) {
  typename FloatFormat<F>::Bits b = static_cast<typename FloatFormat<F>::Bits>(biased) << FloatFormat<F>::kMantissa;
  F v;
  memcpy(&v, &b, sizeof(F));
  return v;
}

template <typename F>
BPL_HOST_DEVICE inline F repeated_sum(F w, uint64_t n) {
  if (n == 0) return F(0);
  const F first = F(0) + w;  // 0 + (-0) is +0; NaN and the infinities stay what they are
  if (!(w == w) || w == F(0) || biased_exponent(w) == FloatFormat<F>::kExpMask) return first;
  if (n <= 16) {  // few addends (the usual count of a spiking network's time step): the loop itself
    F s = first;
    for (uint32_t k = 1; k < static_cast<uint32_t>(n); ++k) s = s + w;
    return s;
  }
  const F a = w < F(0) ? -w : w;  // rounding to nearest is symmetric: sum |w|, restore the sign
  F s = a;
  uint64_t left = n - 1;
  while (left != 0) {
    if (left < 4) {
      s = s + a;
      --left;
      continue;
    }
    const F s1 = s + a, s2 = s1 + a, s3 = s2 + a;
    left -= 3;
    s = s3;
    const uint32_t e = biased_exponent(s3);
    if (e == FloatFormat<F>::kExpMask) break;  // overflowed to infinity, which further additions keep
    if (biased_exponent(s1) != e || biased_exponent(s2) != e) continue;
    const F d = s3 - s2;  // exact: both in one binade
    if (d == F(0)) break;  // w is below half the spacing: the sum no longer moves
    if (e + 1 == FloatFormat<F>::kExpMask) continue;  // the last binade: step by step to infinity
    // steps that certainly end below the top of the binade (the quotient is rounded, hence the margin)
    const F room = (power_of_two<F>(e + 1) - s3) / d;
    if (!(room > F(8))) continue;
    uint64_t j = static_cast<uint64_t>(room) - 4;
    if (j > left) j = left;
    s = s3 + static_cast<F>(j) * d;  // exact: a multiple of the spacing inside the binade
    left -= j;
  }
  return w < F(0) ? -s : s;
}

}  // namespace bpl
