// Generator-stream walker shared by the jitconn kernels: one wave64 walks one std::mt19937
// stream (mt_wave.h) and hands the synapses it finds, 64 lanes at a time, to a callback.
#pragma once

#include <cmath>

#include "common.h"
#include "mt_wave.h"

namespace bpl {

enum : int { kHomo = 0, kUniform = 1, kNormal = 2 };
enum : int { kInEvent = 0, kInDense = 1 };

// weight draws ----------------------------------------------------------------------------------
// std::uniform_real_distribution<T>{a,b} computes canonical * (b - a) + a; the descriptor carries
// a and the range b - a (as the reference's GPU descriptors do, lib/gpu_jitconn_event_matvec.cu:
// 221-222), so the range is formed by the caller.  No contraction.
__device__ __forceinline__ float uniform_weight(const uint32_t *w, float a, float range) {
  return __fadd_rn(__fmul_rn(canonical_f32(w[0]), range), a);
}
__device__ __forceinline__ double uniform_weight(const uint32_t *w, double a, double range) {
  return __dadd_rn(__dmul_rn(canonical_f64(w[0], w[1]), range), a);
}

template <typename T1>
struct WeightWords {
  static constexpr int value = sizeof(T1) == 4 ? 1 : 2;  // mt19937 words per uniform weight
};

// LDS words one wave needs: the generator state.
template <typename T1, int W>
struct StreamLds {
  static constexpr int words = kMtStateWords;
};

__device__ __forceinline__ double read_lane_f64(double v, int l) {
  const unsigned long long b = static_cast<unsigned long long>(__double_as_longlong(v));
  const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b), l));
  const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), l));
  return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}

// Lane l receives lane l - 1's value, across the whole wave, in one data-parallel move (lane 0
// keeps its own); the general shuffle goes through the LDS crossbar and a dozen index instructions.
__device__ __forceinline__ uint32_t wave_shift_up1(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(v), static_cast<int>(v), 0x138 /* wave_shr:1 */,
                                                           0xf, 0xf, false));
}
__device__ __forceinline__ float wave_shift_up1(float v) {
  return __builtin_bit_cast(float, wave_shift_up1(__builtin_bit_cast(uint32_t, v)));
}
__device__ __forceinline__ double wave_shift_up1(double v) {
  const unsigned long long b = static_cast<unsigned long long>(__double_as_longlong(v));
  const uint32_t lo = wave_shift_up1(static_cast<uint32_t>(b)), hi = wave_shift_up1(static_cast<uint32_t>(b >> 32));
  return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}

// std::normal_distribution<float> (libstdc++, Marsaglia polar): candidate pair from two words
struct PolarF32 {
  float x, y, r2;
  bool ok;
};
__device__ __forceinline__ PolarF32 polar_attempt(uint32_t w0, uint32_t w1) {
  PolarF32 a;
  // 2 * canonical - 1: the scalings by powers of two are exact, so one fused multiply-add rounds where
  // the subtraction of the CPU code rounds
  a.x = fmaf(canonical_f32_scaled(w0), 0x1p-31f, -1.0f);
  a.y = fmaf(canonical_f32_scaled(w1), 0x1p-31f, -1.0f);
  a.r2 = __fadd_rn(__fmul_rn(a.x, a.x), __fmul_rn(a.y, a.y));
  a.ok = !(a.r2 > 1.0f || a.r2 == 0.0f);
  return a;
}

// Roles of the 64 two-word units of one batch of a normal-weight stream.  Which units are polar
// attempts and which are skips follows from a small automaton over the units' "this attempt
// would be accepted" bits; it runs on the scalar unit eight units at a time through a table:
// entry [byte of accept bits] holds, for every state the automaton can enter the eight units in
// (one byte per state), the units at which an attempt is accepted and 8 x the state it leaves in.
struct RoleEntry {
  uint32_t accept, next;
};
struct RoleTable {
  RoleEntry e[256];
};
// float: 0 attempt expected, 1 first skip after an accepted attempt, 2 second skip.
// double (kStates == 4; a unit is one coordinate): 0 X expected, 1 Y expected, 2 first skip, 3 second skip.
template <int kStates>
constexpr RoleTable make_role_table() {
  RoleTable t{};
  for (uint32_t b = 0; b < 256; ++b) {
    uint32_t acc = 0, nxt = 0;
    for (int s0 = 0; s0 < kStates; ++s0) {
      int s = s0;
      uint32_t e = 0;
      for (int i = 0; i < 8; ++i) {
        const bool ok = (b >> i) & 1u;
        if (kStates == 3) {
          if (s == 0) {
            if (ok) e |= 1u << i, s = 1;
          } else {
            s = (s == 1) ? 2 : 0;
          }
        } else {
          if (s == 0) s = 1;
          else if (s == 1) {
            if (ok) e |= 1u << i, s = 2;
            else s = 0;
          } else {
            s = (s == 2) ? 3 : 0;
          }
        }
      }
      acc |= e << (8 * s0);
      nxt |= static_cast<uint32_t>(8 * s) << (8 * s0);
    }
    t.e[b].accept = acc;
    t.e[b].next = nxt;
  }
  return t;
}
static __constant__ const RoleTable kRolesF32 = make_role_table<3>();
static __constant__ const RoleTable kRolesF64 = make_role_table<4>();

// accept mask of a batch; `state8` = 8 x automaton state, carried from batch to batch
__device__ __forceinline__ uint64_t accepted_units(const RoleTable &tab, uint64_t okm, uint32_t &state8) {
  uint64_t acc = 0;
  uint32_t sh = state8;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const RoleEntry t = tab.e[static_cast<uint32_t>(okm >> (8 * c)) & 0xffu];
    acc |= static_cast<uint64_t>((t.accept >> sh) & 0xffu) << (8 * c);
    sh = (t.next >> sh) & 0xffu;
  }
  state8 = sh;
  return acc;
}

// Walks stream std::mt19937{stream_seed} over [0, n): calls f(index, weight, valid) once per
// batch with the whole wave converged; `valid` marks the lanes that hold a synapse of the row.
//
// `pre` points at the stream's 624 seeded state words when they were prepared by
// launch_seed_streams(); with nullptr the wave seeds the generator itself on the scalar unit.
//
// `loaded()` is called once, when the generator state is in LDS and `pre` is no longer read.
struct NoLoadHook {
  __device__ __forceinline__ void operator()() const {}
};
template <typename T1, int W, typename F, typename L = NoLoadHook>
__device__ __forceinline__ void walk_stream(uint32_t *st, int lane, uint32_t stream_seed, const uint32_t *pre,
                                            uint32_t n, double log_p_, T1 wa, T1 wb, F &&f, L &&loaded = L()) {
  const SkipParams log_p = make_skip_params(log_p_);
  if (pre != nullptr) mt_load(st, pre, lane);
  else mt_seed(st, stream_seed, lane);
  loaded();
  uint32_t pos = 0;
  // With every skip >= 1 a row ends within n/64 + 1 batches; the cap only guards against a
  // generator state that yields zero skips forever (log_p is validated on the host).
  const uint32_t max_batches = n / 16u + 1024u;
  if constexpr (W == kHomo) {
    // stream: K K K ...   synapse s sits at K_0 + ... + K_s
    uint32_t carry = 0;
    for (uint32_t b = 0; b < max_batches; ++b) {
      uint32_t w[2] = {1u, 1u};
      mt_generate<2>(st, pos, lane, kWave, w);
      const uint32_t skip = skip_from_words(w[0], w[1], log_p);
      const uint32_t idx = carry + wave_inclusive_scan_u32(skip);
      // (the positions rise from lane to lane: the lanes of the row are exactly those below n)
      const bool over = idx >= n;
      const uint64_t done = __ballot(over);
      f(idx, T1(1), !over);
      if (done) break;
      carry = __builtin_amdgcn_readlane(idx, kWave - 1);
    }
  } else if constexpr (W == kUniform) {
    // stream: K  (w K) (w K) ...   synapse s sits at K_0 + ... + K_s, its weight precedes K_{s+1}
    constexpr int WW = WeightWords<T1>::value;
    constexpr int K = WW + 2;
    constexpr int NL = (K == 3) ? 64 : 56;  // K * NL <= 227
    uint32_t w0[2] = {1u, 1u};
    mt_generate<2>(st, pos, lane, 1, w0);
    uint32_t carry = __builtin_amdgcn_readfirstlane(skip_from_words(w0[0], w0[1], log_p));
    for (uint32_t b = 0; b < max_batches; ++b) {
      uint32_t w[K];
#pragma unroll
      for (int i = 0; i < K; ++i) w[i] = 1u;
      mt_generate<K>(st, pos, lane, NL, w);
      const T1 weight = uniform_weight(w, wa, wb);
      uint32_t skip = skip_from_words(w[WW], w[WW + 1], log_p);
      if (lane >= NL) skip = 0;
      const uint32_t incl = wave_inclusive_scan_u32(skip);
      const uint32_t idx = carry + incl - skip;
      const uint64_t done = __ballot(lane < NL && idx >= n);
      const int nvalid = done ? (__ffsll(static_cast<unsigned long long>(done)) - 1) : NL;
      f(idx, weight, lane < nvalid);
      if (done) break;
      carry += __builtin_amdgcn_readlane(incl, kWave - 1);
    }
  } else if constexpr (W == kNormal && sizeof(T1) == 4) {
    // stream in 2-word units: K  (A..A K) (K) (A..A K) (K) ...   A = polar attempt (x word, y word),
    // the last A of a group is the accepted one; the first K after it belongs to the synapse
    // that receives y*mult, the second K to the synapse that receives the cached x*mult.
    // Every lane evaluates its unit both ways; accepted_units() assigns the roles.
    uint32_t w0[2] = {1u, 1u};
    mt_generate<2>(st, pos, lane, 1, w0);
    uint32_t carry = __builtin_amdgcn_readfirstlane(skip_from_words(w0[0], w0[1], log_p));
    uint32_t state8 = 0;
    float prev_x62 = 0.f, prev_x63 = 0.f, prev_y63 = 0.f;
    for (uint32_t b = 0; b < max_batches; ++b) {
      uint32_t w[2] = {1u, 1u};
      mt_generate<2>(st, pos, lane, kWave, w);
      const PolarF32 a = polar_attempt(w[0], w[1]);
      const uint64_t okm = __ballot(a.ok);
      // An accepted attempt at unit q makes q + 1 the first and q + 2 the second skip; a role
      // that falls past unit 63 belongs to the next batch and comes back through `state8`.
      const uint32_t entered = state8;
      const uint64_t acc = accepted_units(kRolesF32, okm, state8);
      const uint64_t k1 = (acc << 1) | (entered == 8u ? 1ull : 0ull);
      const uint64_t k2 = (acc << 2) | (entered == 8u ? 2ull : entered == 16u ? 1ull : 0ull);
      const bool is_k1 = (k1 >> lane) & 1ull;
      const bool is_k2 = (k2 >> lane) & 1ull;
      const bool is_k = is_k1 || is_k2;
      float xw = 0.f, yw = 0.f;
      if (a.ok) {
        const float mult = __fsqrt_rn(__fdiv_rn(__fmul_rn(-2.0f, logf(a.r2)), a.r2));
        xw = __fmul_rn(a.x, mult);
        yw = __fmul_rn(a.y, mult);
      }
      float y_m1 = wave_shift_up1(yw);
      float x_m2 = wave_shift_up1(wave_shift_up1(xw));
      if (lane == 0) y_m1 = prev_y63, x_m2 = prev_x62;
      if (lane == 1) x_m2 = prev_x63;
      const float raw = is_k1 ? y_m1 : x_m2;
      const T1 weight = static_cast<T1>(__fadd_rn(__fmul_rn(raw, static_cast<float>(wb)), static_cast<float>(wa)));
      const uint32_t skip_any = skip_from_words(w[0], w[1], log_p);  // wave-converged call
      const uint32_t skip = is_k ? skip_any : 0u;
      const uint32_t incl = wave_inclusive_scan_u32(skip);
      const uint32_t idx = carry + incl - skip;
      const uint64_t done = __ballot(is_k && idx >= n);
      const int first = done ? (__ffsll(static_cast<unsigned long long>(done)) - 1) : kWave;
      f(idx, weight, is_k && lane < first);
      if (done) break;
      carry += __builtin_amdgcn_readlane(incl, kWave - 1);
      prev_x62 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xw), 62));
      prev_x63 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xw), 63));
      prev_y63 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, yw), 63));
    }
  } else {
    // std::normal_distribution<double>: every draw is one canonical double, so the stream again
    // consists of 2-word units:  K  (X Y .. X Y K) (K) (X Y .. X Y K) (K) ...   X, Y = the two
    // coordinates of a polar attempt, the last pair of a group is the accepted one; the first K
    // after it belongs to the synapse that receives y*mult, the second K to the synapse that
    // receives the cached x*mult.  Every lane evaluates its unit as a coordinate (and, with its
    // left neighbour's, as the end of an attempt) and as a skip; accepted_units() assigns the roles.
    uint32_t w0[2] = {1u, 1u};
    mt_generate<2>(st, pos, lane, 1, w0);
    uint32_t carry = __builtin_amdgcn_readfirstlane(skip_from_words(w0[0], w0[1], log_p));
    uint32_t state8 = 0;
    double prev_v63 = 0.0, prev_x62 = 0.0, prev_x63 = 0.0, prev_y63 = 0.0;
    for (uint32_t b = 0; b < max_batches; ++b) {
      uint32_t w[2] = {1u, 1u};
      mt_generate<2>(st, pos, lane, kWave, w);
      const double v = __dsub_rn(__dmul_rn(2.0, canonical_f64(w[0], w[1])), 1.0);
      double v_m1 = wave_shift_up1(v);
      if (lane == 0) v_m1 = prev_v63;
      const double r2 = __dadd_rn(__dmul_rn(v_m1, v_m1), __dmul_rn(v, v));
      const bool ok = !(r2 > 1.0 || r2 == 0.0);  // an attempt (lane - 1, lane) would be accepted
      const uint64_t okm = __ballot(ok);
      // unit 0 may complete the attempt begun by the previous batch's last unit (state 1)
      const uint32_t entered = state8;
      const uint64_t acc = accepted_units(kRolesF64, okm, state8);
      const uint64_t k1 = (acc << 1) | (entered == 16u ? 1ull : 0ull);
      const uint64_t k2 = (acc << 2) | (entered == 16u ? 2ull : entered == 24u ? 1ull : 0ull);
      const bool is_k1 = (k1 >> lane) & 1ull;
      const bool is_k2 = (k2 >> lane) & 1ull;
      const bool is_k = is_k1 || is_k2;
      double xw = 0.0, yw = 0.0;
      if (ok) {
        const double mult = sqrt(-2 * log(r2) / r2);
        xw = __dmul_rn(v_m1, mult);
        yw = __dmul_rn(v, mult);
      }
      double y_m1 = wave_shift_up1(yw);
      double x_m2 = wave_shift_up1(wave_shift_up1(xw));
      if (lane == 0) y_m1 = prev_y63, x_m2 = prev_x62;
      if (lane == 1) x_m2 = prev_x63;
      const double raw = is_k1 ? y_m1 : x_m2;
      const T1 weight = static_cast<T1>(__dadd_rn(__dmul_rn(raw, static_cast<double>(wb)), static_cast<double>(wa)));
      const uint32_t skip_any = skip_from_words(w[0], w[1], log_p);  // wave-converged call
      const uint32_t skip = is_k ? skip_any : 0u;
      const uint32_t incl = wave_inclusive_scan_u32(skip);
      const uint32_t idx = carry + incl - skip;
      const uint64_t done = __ballot(is_k && idx >= n);
      const int first = done ? (__ffsll(static_cast<unsigned long long>(done)) - 1) : kWave;
      f(idx, weight, is_k && lane < first);
      if (done) break;
      carry += __builtin_amdgcn_readlane(incl, kWave - 1);
      prev_v63 = read_lane_f64(v, kWave - 1);
      prev_x62 = read_lane_f64(xw, kWave - 2);
      prev_x63 = read_lane_f64(xw, kWave - 1);
      prev_y63 = read_lane_f64(yw, kWave - 1);
    }
  }
}

// Seeds `count` generators std::mt19937{seed + first + i} and stores their 624-word states at
// states[i * 624].  One lane per stream: the 623-step recurrence of 64 streams advances in
// lock step on the vector unit, and LDS transposes 64 x 64 tiles so that every state is written
// with contiguous 256-byte stores.  The scalar unit (one per CU) can seed only one stream per
// wave at a time and saturates when every row of a large matrix needs its own generator.
void launch_seed_streams(hipStream_t stream, uint32_t seed, uint32_t first, uint32_t count, uint32_t *states);

// Streams seeded per launch_seed_streams() call by the operators that use it, and the number
// of streams from which they do.
constexpr uint32_t kSeedChunk = 131072;
constexpr uint32_t kSeedAheadMin = 8192;

}  // namespace bpl
