// jitconn event matvec with the stateless ("hash") connectivity of the reference's first kernel
// generation: the targets gpu_event_matvec_prob_{homo,uniform,normal}_{float,double}.
//
//   buffers = [event_ids int32[n_col] (the positions of the events, as `nonzero_*` lists them),
//              event_num int32[1], out T[n_row]]
//   opaque  = bpl_jitconn_prob_homo_descriptor / bpl_jitconn_prob_weight_descriptor whose field
//             `log_p` carries the connection probability itself here (not a logarithm), as the
//             reference's descriptors of these targets do (their field is called `prob`)
//
// Synapse (row, col) exists iff lfsr113(seed + n_col * row + col) * 2^-32 < prob, all in 32-bit
// wrapping arithmetic; its weight is 1 (homo: the caller multiplies), taus88 * w_range + w_min
// (uniform) or w_mu + sqrt(-2 log u) cos(2 pi v) * w_sigma with (u, v) two consecutive taus88
// outputs (normal).  out[row] sums the weights of the row's synapses to the listed event
// columns, in the order of the list, in T (each addend formed in double and added to the
// widened sum, as `sum += expr` with a float `sum` does).
//
// Follows lib/gpu_jitconn_event_matvec.cu:10-51 (homo), :138-183 (uniform), :281-331 (normal),
// launchers :53-79, :186-215, :334-362, exports :432-450, and the generators of
// lib/kernel_helpers_random.cuh:12-71.  The reference's Python layer builds only the _v2 names
// (brainpylib/_src/jitconn_ops/event_matvec.py:224,367,513); these six targets are reachable
// through the registration table alone, there as here.
//
// One lane per output row; the event list goes through LDS in tiles, so every lane of a wave
// reads the same word (a broadcast).  lfsr113 * 2^-32 < prob is decided in integers:
// z * 2^-32 < prob  <=>  z < prob * 2^32 (scaling by a power of two is exact)  <=>  z < ceil(prob * 2^32).
#include <cmath>

#include "common.h"
#include "targets.h"

namespace bpl {
namespace {

enum : int { kHomo = 0, kUniform = 1, kNormal = 2 };
constexpr int kHashThreads = 256;
constexpr int kHashTile = 1024;  // event ids staged in LDS at a time

// one step of L'Ecuyer's LFSR113 from the state (s + 1, s + 7, s + 15, s + 127): the 32-bit output
__device__ __forceinline__ uint32_t lfsr113_word(uint32_t s) {
  uint32_t z1 = s + 1u, z2 = s + 7u, z3 = s + 15u, z4 = s + 127u, b;
  b = ((z1 << 6) ^ z1) >> 13;
  z1 = ((z1 & 4294967294u) << 18) ^ b;
  b = ((z2 << 2) ^ z2) >> 27;
  z2 = ((z2 & 4294967288u) << 2) ^ b;
  b = ((z3 << 13) ^ z3) >> 21;
  z3 = ((z3 & 4294967280u) << 7) ^ b;
  b = ((z4 << 3) ^ z4) >> 12;
  z4 = ((z4 & 4294967168u) << 13) ^ b;
  return z1 ^ z2 ^ z3 ^ z4;
}

// one step of taus88 on (s1, s2, s3): the 32-bit output
__device__ __forceinline__ uint32_t taus88_step(uint32_t &s1, uint32_t &s2, uint32_t &s3) {
  uint32_t b;
  b = ((s1 << 13) ^ s1) >> 19;
  s1 = ((s1 & 4294967294u) << 12) ^ b;
  b = ((s2 << 2) ^ s2) >> 25;
  s2 = ((s2 & 4294967288u) << 4) ^ b;
  b = ((s3 << 3) ^ s3) >> 11;
  s3 = ((s3 & 4294967280u) << 17) ^ b;
  return s1 ^ s2 ^ s3;
}

constexpr double kTwoPow32Inv = 2.3283064365386963e-10;  // 2^-32

template <typename T, int W>
__global__ __launch_bounds__(kHashThreads) void event_matvec_hash_kernel(const int32_t *__restrict__ event_ids,
                                                                         const int32_t *__restrict__ event_num,
                                                                         uint32_t seed, uint64_t threshold, double w_a,
                                                                         double w_b, uint32_t n_row, uint32_t n_col,
                                                                         T *__restrict__ out) {
  __shared__ int32_t s_ids[kHashTile];
  int64_t n64 = event_num[0];
  if (n64 < 0) n64 = 0;
  if (n64 > n_col) n64 = n_col;  // the list has n_col entries
  const uint32_t n = static_cast<uint32_t>(n64);
  const uint32_t row = blockIdx.x * kHashThreads + threadIdx.x;
  const uint32_t base = seed + n_col * row;
  T sum = T(0);
  for (uint32_t t0 = 0; t0 < n; t0 += kHashTile) {
    const uint32_t m = (n - t0 < kHashTile) ? n - t0 : kHashTile;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < m; i += kHashThreads) s_ids[i] = event_ids[t0 + i];
    __syncthreads();
    for (uint32_t i = 0; i < m; ++i) {
      const uint32_t s = base + static_cast<uint32_t>(s_ids[i]);
      if (lfsr113_word(s) < threshold) {
        if (W == kHomo) {
          sum += T(1);
        } else {
          uint32_t s1 = s + 1u, s2 = s + 7u, s3 = s + 15u;
          const double u = taus88_step(s1, s2, s3) * kTwoPow32Inv;
          double w;
          if (W == kUniform) {
            w = fma(u, w_b, w_a);  // (the reference's compiler contracts u * w_range + w_min)
          } else {
            const double v = taus88_step(s1, s2, s3) * kTwoPow32Inv;
            w = fma(sqrt(-2 * log(u)) * cos(2 * M_PI * v), w_b, w_a);
          }
          sum = static_cast<T>(static_cast<double>(sum) + w);
        }
      }
    }
  }
  if (row < n_row) out[row] = sum;
}

// smallest integer t with z < t  <=>  z * 2^-32 < prob, for 32-bit z
uint64_t hash_threshold(double prob) {
  if (!(prob > 0.0)) return 0;  // also NaN: no synapse
  const double scaled = prob * 4294967296.0;
  if (scaled >= 4294967296.0) return 1ull << 32;
  return static_cast<uint64_t>(std::ceil(scaled));
}

template <typename T, int W, typename D>
void hash_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t opaque_len) {
  D d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  if (d.n_row == 0) return;
  double w_a = 0.0, w_b = 0.0;
  if constexpr (W != kHomo) w_a = d.w_a, w_b = d.w_b;
  hipLaunchKernelGGL((event_matvec_hash_kernel<T, W>), dim3(div_up(d.n_row, kHashThreads)), dim3(kHashThreads), 0, stream,
                     static_cast<const int32_t *>(buffers[0]), static_cast<const int32_t *>(buffers[1]), d.seed,
                     hash_threshold(d.log_p), w_a, w_b, d.n_row, d.n_col, static_cast<T *>(buffers[2]));
  check_launch(target);
}

}  // namespace
}  // namespace bpl

using namespace bpl;

#define BPL_DEFINE(name, T, W, D)                                                                  \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    hash_entry<T, W, D>(__func__, static_cast<hipStream_t>(stream), buffers, opaque, opaque_len);   \
  }

BPL_DEFINE(gpu_event_matvec_prob_homo_float, float, kHomo, bpl_jitconn_prob_homo_descriptor)
BPL_DEFINE(gpu_event_matvec_prob_homo_double, double, kHomo, bpl_jitconn_prob_homo_descriptor)
BPL_DEFINE(gpu_event_matvec_prob_uniform_float, float, kUniform, bpl_jitconn_prob_weight_descriptor)
BPL_DEFINE(gpu_event_matvec_prob_uniform_double, double, kUniform, bpl_jitconn_prob_weight_descriptor)
BPL_DEFINE(gpu_event_matvec_prob_normal_float, float, kNormal, bpl_jitconn_prob_weight_descriptor)
BPL_DEFINE(gpu_event_matvec_prob_normal_double, double, kNormal, bpl_jitconn_prob_weight_descriptor)
