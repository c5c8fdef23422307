/*
 * CPU oracle for the event-driven sparse operator path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference's CPU backend so that the
 * HIP kernels can be checked against them on identical inputs.  It is never linked into,
 * loaded by or called from the shipped library; only tests, the smoke check and the
 * benchmark's CPU-baseline leg may use it.
 *
 * Each function cites the reference source it follows (paths relative to the reference
 * tree).  Third-party arithmetic the reference relies on and which is restated here:
 *   - std::mt19937 (ISO C++ [rand.eng.mers]; standard-exact, pinned by the 10000th-output
 *     known answer 4123659995 for the default seed 5489),
 *   - libstdc++ (GCC 11.4) generate_canonical / uniform_real_distribution /
 *     normal_distribution (Marsaglia polar, second variate cached), which are
 *     implementation-defined; pinned bit-for-bit against the reference's own sources
 *     compiled with that libstdc++,
 *   - glibc log/ceil/logf/sqrtf, used directly.
 *
 * Parity status of every exported function is listed in oracle/__init__.py next to its
 * Python binding.
 */
#define _GNU_SOURCE /* M_PI */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------ */
/* threads for the loops the reference runs under numba.prange                                 */
/* ------------------------------------------------------------------------------------------ */
static int g_threads = 1;

ORACLE_API void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
ORACLE_API int oracle_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------------------------------ */
/* std::mt19937                                                                                */
/* ------------------------------------------------------------------------------------------ */
typedef struct {
  uint32_t mt[624];
  int pos;
} mt19937_t;

static void mt_seed(mt19937_t *g, uint32_t seed) {
  g->mt[0] = seed;
  for (uint32_t i = 1; i < 624; ++i) {
    uint32_t x = g->mt[i - 1];
    g->mt[i] = 1812433253u * (x ^ (x >> 30)) + i;
  }
  g->pos = 624;
}

static void mt_refill(mt19937_t *g) {
  uint32_t *mt = g->mt;
  for (int k = 0; k < 624; ++k) {
    uint32_t y = (mt[k] & 0x80000000u) | (mt[(k + 1) % 624] & 0x7fffffffu);
    mt[k] = mt[(k + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
  }
  g->pos = 0;
}

static inline uint32_t mt_next(mt19937_t *g) {
  if (g->pos >= 624) mt_refill(g);
  uint32_t y = g->mt[g->pos++];
  y ^= y >> 11;
  y ^= (y << 7) & 0x9d2c5680u;
  y ^= (y << 15) & 0xefc60000u;
  y ^= y >> 18;
  return y;
}

/* libstdc++ generate_canonical<double,53>(mt19937): two words, low word first; the 64-bit
 * sum is rounded once to double, then divided by 2^64 (exact); 1.0 is clamped. */
static inline double canon_f64(mt19937_t *g) {
  double lo = (double)mt_next(g);
  double hi = (double)mt_next(g);
  double r = (lo + hi * 4294967296.0) / 18446744073709551616.0;
  if (r >= 1.0) r = nextafter(1.0, 0.0);
  return r;
}

/* libstdc++ generate_canonical<float,24>(mt19937): one word rounded to float, / 2^32. */
static inline float canon_f32(mt19937_t *g) {
  float r = (float)mt_next(g) / 4294967296.0f;
  if (r >= 1.0f) r = nextafterf(1.0f, 0.0f);
  return r;
}

/* (unsigned int) of a double the way x86-64 gcc compiles it: cvttsd2si to 64 bits, keep the
 * low 32; out-of-range and NaN give the "integer indefinite" value whose low half is 0. */
static inline uint32_t f64_to_u32(double x) {
  if (!(x > -9223372036854775808.0 && x < 9223372036854775808.0)) return 0u;
  return (uint32_t)(uint64_t)(int64_t)x;
}

/* one geometric skip: (unsigned) ceil(log(U) / log_p), U from uniform_real_distribution<double>{0,1}
 * reference: lib/cpu_jitconn_event_matvec.cpp:24,29 */
static inline uint32_t skip_draw(mt19937_t *g, double log_p) {
  return f64_to_u32(ceil(log(canon_f64(g)) / log_p));
}

/* normal_distribution<T> state (libstdc++ caches the second polar variate) */
typedef struct {
  int has_saved;
  float saved_f32;
  double saved_f64;
} normal_state_t;

static inline float uniform_w_f32(mt19937_t *g, float a, float b) {
  return canon_f32(g) * (b - a) + a; /* uniform_real_distribution<float>::operator() */
}
static inline double uniform_w_f64(mt19937_t *g, double a, double b) {
  return canon_f64(g) * (b - a) + a;
}

static inline float normal_w_f32(mt19937_t *g, normal_state_t *s, float mu, float sigma) {
  float ret;
  if (s->has_saved) {
    s->has_saved = 0;
    ret = s->saved_f32;
  } else {
    float x, y, r2;
    do {
      x = (float)((double)(2.0f * canon_f32(g)) - 1.0);
      y = (float)((double)(2.0f * canon_f32(g)) - 1.0);
      r2 = x * x + y * y;
    } while (r2 > 1.0f || r2 == 0.0f);
    float mult = sqrtf(-2 * logf(r2) / r2);
    s->saved_f32 = x * mult;
    s->has_saved = 1;
    ret = y * mult;
  }
  return ret * sigma + mu;
}

static inline double normal_w_f64(mt19937_t *g, normal_state_t *s, double mu, double sigma) {
  double ret;
  if (s->has_saved) {
    s->has_saved = 0;
    ret = s->saved_f64;
  } else {
    double x, y, r2;
    do {
      x = 2.0 * canon_f64(g) - 1.0;
      y = 2.0 * canon_f64(g) - 1.0;
      r2 = x * x + y * y;
    } while (r2 > 1.0 || r2 == 0.0);
    double mult = sqrt(-2 * log(r2) / r2);
    s->saved_f64 = x * mult;
    s->has_saved = 1;
    ret = y * mult;
  }
  return ret * sigma + mu;
}

/* raw generator access so tests can pin the restatement against known answers */
ORACLE_API void oracle_mt19937_words(uint32_t seed, uint32_t skip, uint32_t n, uint32_t *out) {
  mt19937_t g;
  mt_seed(&g, seed);
  for (uint32_t i = 0; i < skip; ++i) (void)mt_next(&g);
  for (uint32_t i = 0; i < n; ++i) out[i] = mt_next(&g);
}
ORACLE_API void oracle_canonical_f64(uint32_t seed, uint32_t n, double *out) {
  mt19937_t g;
  mt_seed(&g, seed);
  for (uint32_t i = 0; i < n; ++i) out[i] = canon_f64(&g);
}
ORACLE_API void oracle_canonical_f32(uint32_t seed, uint32_t n, float *out) {
  mt19937_t g;
  mt_seed(&g, seed);
  for (uint32_t i = 0; i < n; ++i) out[i] = canon_f32(&g);
}
ORACLE_API void oracle_normal_f32(uint32_t seed, float mu, float sigma, uint32_t n, float *out) {
  mt19937_t g;
  normal_state_t s = {0, 0.f, 0.};
  mt_seed(&g, seed);
  for (uint32_t i = 0; i < n; ++i) out[i] = normal_w_f32(&g, &s, mu, sigma);
}
ORACLE_API void oracle_normal_f64(uint32_t seed, double mu, double sigma, uint32_t n, double *out) {
  mt19937_t g;
  normal_state_t s = {0, 0.f, 0.};
  mt_seed(&g, seed);
  for (uint32_t i = 0; i < n; ++i) out[i] = normal_w_f64(&g, &s, mu, sigma);
}

/* ------------------------------------------------------------------------------------------ */
/* Connectivity of one generator stream (the index set the jitconn operators imply).           */
/* Walks one stream seeded with `seed`: first = skip, next += skip, stop at >= n.              */
/* Returns the number of indices; writes at most `cap` of them.                                */
/* reference: lib/cpu_jitconn_event_matvec.cpp:24-30 (the loop with the event test removed)    */
/* ------------------------------------------------------------------------------------------ */
ORACLE_API uint32_t oracle_jitconn_stream_indices(uint32_t seed, double log_p, uint32_t n,
                                                  uint32_t *out, uint32_t cap) {
  mt19937_t g;
  mt_seed(&g, seed);
  uint32_t cnt = 0;
  uint32_t c = skip_draw(&g, log_p);
  while (c < n) {
    if (cnt < cap) out[cnt] = c;
    ++cnt;
    c += skip_draw(&g, log_p);
  }
  return cnt;
}

/* ------------------------------------------------------------------------------------------ */
/* jitconn (event) matvec: instantiated for T in {float,double} x event type                   */
/* ------------------------------------------------------------------------------------------ */
#define W_HOMO 0
#define W_UNIFORM 1
#define W_NORMAL 2

/* float results */
#define T1 float
#define T1SUF f32
#define UNIFORM_W uniform_w_f32
#define NORMAL_W normal_w_f32
#include "jitconn_body.inc"
#undef T1
#undef T1SUF
#undef UNIFORM_W
#undef NORMAL_W

/* double results */
#define T1 double
#define T1SUF f64
#define UNIFORM_W uniform_w_f64
#define NORMAL_W normal_w_f64
#include "jitconn_body.inc"
#undef T1
#undef T1SUF
#undef UNIFORM_W
#undef NORMAL_W

/* ------------------------------------------------------------------------------------------ */
/* CSR operators                                                                               */
/* ------------------------------------------------------------------------------------------ */
#define T1 float
#define T1SUF f32
#include "csr_body.inc"
#undef T1
#undef T1SUF

#define T1 double
#define T1SUF f64
#include "csr_body.inc"
#undef T1
#undef T1SUF

#include "hash_body.inc"

/* ------------------------------------------------------------------------------------------ */
/* event_info: ordered compaction of the nonzero positions, padded with -1, plus the count     */
/* reference: brainpylib/_src/event_ops/event_info_collection.py:143-155                       */
/* elem_size/kind: 0 bool(1 byte), 1 int32, 2 int64, 3 float, 4 double                         */
/* ------------------------------------------------------------------------------------------ */
ORACLE_API void oracle_event_info(const void *events, int kind, uint32_t size, int32_t *ids,
                                  int32_t *num) {
  int32_t n = 0;
  for (uint32_t i = 0; i < size; ++i) ids[i] = -1;
  for (uint32_t i = 0; i < size; ++i) {
    int on;
    switch (kind) {
      case 0: on = ((const uint8_t *)events)[i] != 0; break;
      case 1: on = ((const int32_t *)events)[i] != 0; break;
      case 2: on = ((const int64_t *)events)[i] != 0; break;
      case 3: on = ((const float *)events)[i] != 0.0f; break;
      default: on = ((const double *)events)[i] != 0.0; break;
    }
    if (on) ids[n++] = (int32_t)i;
  }
  num[0] = n;
}
