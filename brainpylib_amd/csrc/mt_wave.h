// A std::mt19937 stream generated cooperatively by one wave64, state in LDS.
//
// The jitconn operators draw one generator stream per output row (or per input column):
// stream i is std::mt19937{seed + i}, the generator of the reference's CPU backend
// (lib/cpu_jitconn_event_matvec.cpp:20-21), restarted per stream the way the reference's GPU
// backend restarts its generator per row (lib/gpu_jitconn_event_matvec.cu:94-96).  A row is
// then exactly what the reference CPU code produces for a one-row matrix seeded `seed + i`.
//
// MT19937 produces word t from words t-624, t-623 and t-227, so up to 227 consecutive words can
// be produced at once from the previous 624: each lane computes K consecutive words
// (64*K <= 227) of the next batch and the 624-word state is a circular buffer in LDS, followed by
// a copy of its first kMtMirror words so that a lane's run of consecutive words never wraps.
// Seeding is a serial 623-step recurrence; it runs on the scalar unit (the seed is wave
// uniform) and the values are packed 64 at a time into a vector register with v_writelane.
#pragma once

#include "common.h"

namespace bpl {

constexpr int kMtN = 624;
constexpr int kMtM = 397;
constexpr int kMtMirror = 4;        // st[624 + i] repeats st[i]: runs of up to 5 words from any slot are contiguous
constexpr int kMtStateWords = kMtN + kMtMirror;  // LDS words reserved per wave

__device__ __forceinline__ void mt_seed(uint32_t *st, uint32_t seed, int lane) {
  uint32_t x = __builtin_amdgcn_readfirstlane(seed);
#pragma unroll 1
  for (int base = 0; base < kMtN; base += kWave) {
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < kWave; ++i) {
      // lane i of v <- x  (x lives in a scalar register)
      asm volatile("v_writelane_b32 %0, %1, %2" : "+v"(v) : "s"(x), "n"(i));
      x = 1812433253u * (x ^ (x >> 30)) + static_cast<uint32_t>(base + i + 1);
    }
    if (base + lane < kMtN) st[base + lane] = v;
    if (base == 0 && lane < kMtMirror) st[kMtN + lane] = v;
  }
}

// Copies a state seeded elsewhere (624 words at `src`) into the wave's LDS buffer.
__device__ __forceinline__ void mt_load(uint32_t *st, const uint32_t *__restrict__ src, int lane) {
#pragma unroll
  for (int base = 0; base < kMtN; base += kWave)
    if (base + lane < kMtN) st[base + lane] = src[base + lane];
  if (lane < kMtMirror) st[kMtN + lane] = src[lane];
}

// Seeds 64 generators at once, lane l the stream std::mt19937{lane_seed}, and stores the states of
// the first n_streams of them at dst[l * 624 .. + 624).  The 623-step recurrence of the 64 streams
// advances in lock step on the vector unit (a few dozen instructions per stream instead of the
// scalar unit's 3,100 for one); every eight steps the words pass through `tile` (LDS of the calling
// wave, 8 x 65 words) so that they leave as 32-byte runs per stream instead of 4-byte words 2,496
// bytes apart.  (Plain stores: the states are read back soon, by waves of the same workgroup, and do
// best when they stay in the L2; with nontemporal stores and loads the 1e6-row walk took 3.6 instead
// of 3.1 ms.)
constexpr int kMtSeedTileWords = 8 * (kWave + 1);
__device__ __forceinline__ void mt_seed_batch(uint32_t *tile, int lane, uint32_t lane_seed, uint32_t *__restrict__ dst,
                                              uint32_t n_streams = kWave) {
  uint32_t x = lane_seed;
  const uint32_t sub = static_cast<uint32_t>(lane) >> 2, pair = static_cast<uint32_t>(lane) & 3u;  // stream within 16, word pair
  uint2 *out = reinterpret_cast<uint2 *>(dst + static_cast<size_t>(sub) * kMtN) + pair;
  // The words of a tile are read back from LDS at the end of a round and stored at the start of the next
  // one, behind its eight steps of the recurrence, so that the chain of multiplications does not wait for
  // the LDS (a wave's LDS operations complete in order: the next round's writes cannot overtake the reads).
  uint2 v[4];
#pragma unroll 1
  for (uint32_t w0 = 0; w0 < kMtN; w0 += 8) {
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
      tile[i * (kWave + 1) + lane] = x;  // word w0 + i of stream `lane`
      x = 1812433253u * (x ^ (x >> 30)) + (w0 + i + 1);
    }
    __builtin_amdgcn_wave_barrier();
    if (w0 != 0) {
#pragma unroll
      for (uint32_t q = 0; q < 4; ++q)  // streams 16 q + sub: words w0 - 8 + 2 pair, + 1
        if (16u * q + sub < n_streams) out[(static_cast<size_t>(16u * q) * kMtN + (w0 - 8u)) / 2u] = v[q];
    }
#pragma unroll
    for (uint32_t q = 0; q < 4; ++q) {
      const uint32_t s = 16u * q + sub;
      v[q].x = tile[(2u * pair) * (kWave + 1) + s];
      v[q].y = tile[(2u * pair + 1u) * (kWave + 1) + s];
    }
    __builtin_amdgcn_wave_barrier();
  }
#pragma unroll
  for (uint32_t q = 0; q < 4; ++q)
    if (16u * q + sub < n_streams) out[(static_cast<size_t>(16u * q) * kMtN + (kMtN - 8u)) / 2u] = v[q];
}

// gfx950 evaluates any function of three words bit by bit in one instruction; 0x6c is (a & c) ^ b,
// 0x96 is a ^ b ^ c (the compiler finds the first only now and then).
__device__ __forceinline__ uint32_t and_xor(uint32_t a, uint32_t c, uint32_t b) {
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x6c);
}

__device__ __forceinline__ uint32_t mt_twist(uint32_t a, uint32_t b, uint32_t c) {
  // y = (a & 0x80000000) | (b & 0x7fffffff) in one bit-field insert (the compiler makes two instructions of it)
  uint32_t y;
  asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(y) : "s"(0x7fffffffu), "v"(b), "v"(a));
  const uint32_t odd = static_cast<uint32_t>(-static_cast<int32_t>(b & 1u));  // all ones when y is odd
  return and_xor(odd, 0x9908b0dfu, c) ^ (y >> 1);
}

__device__ __forceinline__ uint32_t mt_temper(uint32_t y) {
  y ^= y >> 11;
  y = and_xor(y << 7, 0x9d2c5680u, y);
  y = and_xor(y << 15, 0xefc60000u, y);
  y ^= y >> 18;
  return y;
}

// Produces the next K * nlanes words of the stream; lane l < nlanes receives words
// K*l .. K*l + K-1 of them (tempered) in w[].  `pos` is the state slot of the first new word
// (wave uniform, < 624) and is advanced.  Requires K * nlanes <= 227.
//
// A lane reads the K + 1 old words from its first slot s on and the K words from slot
// (s + 397) mod 624 on, and writes K new words from s on: with the first kMtMirror words repeated
// behind the 624th, all three runs are contiguous (s + K <= 627), and only a batch that touches
// the first words or runs past the 624th (a wave-uniform test on `pos`) has copies to keep equal.
template <int K>
__device__ __forceinline__ void mt_generate(uint32_t *st, uint32_t &pos, int lane, int nlanes, uint32_t (&w)[K]) {
  static_assert(K >= 1 && K <= kMtMirror, "words per lane");
  const uint32_t span = static_cast<uint32_t>(K * nlanes);
  if (lane < nlanes) {
    uint32_t s = pos + static_cast<uint32_t>(K * lane);
    s = min(s, s - kMtN);  // (unsigned: s - 624 wraps to a huge value while s < 624)
    uint32_t f = s + kMtM;
    f = min(f, f - kMtN);
    uint32_t near_[K + 1], far_[K], fresh[K];
#pragma unroll
    for (int i = 0; i <= K; ++i) near_[i] = st[s + i];
#pragma unroll
    for (int i = 0; i < K; ++i) far_[i] = st[f + i];
#pragma unroll
    for (int i = 0; i < K; ++i) {
      fresh[i] = mt_twist(near_[i], near_[i + 1], far_[i]);
      st[s + i] = fresh[i];
      w[i] = mt_temper(fresh[i]);
    }
    if (pos < static_cast<uint32_t>(kMtMirror) || pos + span > static_cast<uint32_t>(kMtN)) {
#pragma unroll
      for (int i = 0; i < K; ++i) {
        const uint32_t a = s + i;
        if (a >= kMtN) st[a - kMtN] = fresh[i];
        else if (a < static_cast<uint32_t>(kMtMirror)) st[a + kMtN] = fresh[i];
      }
    }
  }
  pos += span;
  if (pos >= kMtN) pos -= kMtN;
}

// libstdc++ generate_canonical<double,53>(mt19937): low word first, the 64-bit sum rounded once
// to double, scaled by 2^-64, clamped below 1.
__device__ __forceinline__ double canonical_f64(uint32_t lo, uint32_t hi) {
  const double s = __dadd_rn(static_cast<double>(lo), __dmul_rn(static_cast<double>(hi), 4294967296.0));
  const double r = s * 0x1p-64;  // exact scaling
  return r >= 1.0 ? 0x1.fffffffffffffp-1 : r;  // nextafter(1, 0)
}

// libstdc++ generate_canonical<float,24>(mt19937): one word rounded to float, scaled by 2^-32, and a
// result of 1 replaced by nextafterf(1, 0).  The word rounds up to 2^32 from 0xffffff80 on, and every
// word from 0xffffff00 to 0xffffff7f rounds to 0xffffff00 = nextafterf(1, 0) * 2^32: capping the WORD
// at 0xffffff7f gives the same floats with one integer minimum instead of a compare and a select.
__device__ __forceinline__ float canonical_f32_scaled(uint32_t word) {  // canonical * 2^32
  return static_cast<float>(min(word, 0xffffff7fu));
}
__device__ __forceinline__ float canonical_f32(uint32_t word) { return canonical_f32_scaled(word) * 0x1p-32f; }

// (unsigned int) of a double as x86-64 compiles it: truncate to int64, keep the low 32 bits;
// out of range and NaN give 0.
__device__ __forceinline__ uint32_t f64_to_u32_x86(double x) {
  if (x >= 0.0 && x < 4294967296.0) return static_cast<uint32_t>(x);  // the only case seen in practice
  if (!(x > -9223372036854775808.0 && x < 9223372036854775808.0)) return 0u;
  return static_cast<uint32_t>(static_cast<uint64_t>(static_cast<long long>(x)));
}

// Parameters of the skip computation, derived once per kernel from log_p.
struct SkipParams {
  double log_p;      // log(1 - p)
  double inv_log2;   // ln(2) / log_p: skip = ceil(log2(U) * inv_log2)
  double offset;     // 1 - 32 * inv_log2: the fast path works on log2(U * 2^32) and truncates instead of ceil()
  double safe_half;  // the fast path is trusted while |frac(q) - 1/2| < safe_half = 1/2 - guard
};

// Error of the fast path's log2(U): U * 2^32 is formed in fp32 from the two words (two roundings,
// 2^-23 relative, 1.72e-7 on the logarithm) and the hardware fp32 log2 of its mantissa in [0.5, 1) is
// documented to 1 ulp, 2^-24 = 5.96e-8 on a result in [-1, 0] (bpl_selfcheck_jitconn_skips measures
// it over all 2^23 mantissas): 2.32e-7 together, the rest is margin.
constexpr double kSkipLog2Error = 3e-7;

__device__ __forceinline__ SkipParams make_skip_params(double log_p) {
  SkipParams sp;
  sp.log_p = log_p;
  sp.inv_log2 = 0.6931471805599453094 / log_p;
  sp.offset = 1.0 - 32.0 * sp.inv_log2;
  // The quotient is off by at most kSkipLog2Error * |inv_log2| plus fp64 rounding; inside that band
  // around an integer the exact path decides.  Quotients that could leave the range of uint32
  // (log2(U) >= -64): always the exact path, which converts as x86-64 does.
  const double guard = kSkipLog2Error * fabs(sp.inv_log2) + 1e-9;
  sp.safe_half = (fabs(sp.inv_log2) * 64.0 + 2.0 < 4.0e9) ? 0.5 - guard : -1.0;
  return sp;
}

// One geometric skip: (unsigned) ceil(log(U) / log_p)  (lib/cpu_jitconn_event_matvec.cpp:24),
// U = canonical double of two generator words (low word first).
//
// Exact path: fp64 log and IEEE division, as the CPU code.
__device__ __forceinline__ uint32_t skip_exact(uint32_t lo, uint32_t hi, const SkipParams &sp) {
  return f64_to_u32_x86(ceil(log(canonical_f64(lo, hi)) / sp.log_p));
}

// Fast path: log2(U * 2^32) = exponent + v_log_f32(mantissa) of the fp32 value of the two words, one
// fused multiply-add to q + 1 = log2(U) * inv_log2 + 1, truncation.  `safe` says that q is further
// than the guard from an integer, i.e. that no rounding of the exact path could land on another
// ceil() (not so for q = inf or NaN, U = 0).
__device__ __forceinline__ uint32_t skip_fast(uint32_t lo, uint32_t hi, const SkipParams &sp, bool &safe) {
  const float f = fmaf(static_cast<float>(lo), 0x1p-32f, static_cast<float>(hi));
  int e;
  const float m = frexpf(f, &e);  // f = m * 2^e, m in [0.5, 1)
  const double l2 = static_cast<double>(e) + static_cast<double>(__log2f(m));
  const double q1 = fma(l2, sp.inv_log2, sp.offset);
  safe = fabs(__builtin_amdgcn_fract(q1) - 0.5) < sp.safe_half;
  return static_cast<uint32_t>(q1);
}

// If any lane of the wave is inside the band, the whole wave takes the exact path (a wave-uniform
// branch); for conn_prob around 1e-3 that happens in a few per cent of the batches, for very sparse
// matrices (guard >= 0.5) always.
__device__ __forceinline__ uint32_t skip_from_words(uint32_t lo, uint32_t hi, const SkipParams &sp) {
  bool safe;
  const uint32_t fast = skip_fast(lo, hi, sp, safe);
  if (__ballot(!safe) == 0) return fast;
  return skip_exact(lo, hi, sp);
}

}  // namespace bpl
