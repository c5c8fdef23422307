// jitconn matmat for gfx950:  Y[m,n] = X[m,k] @ M[k,n],  M regenerated on the fly.
//
// Column j of M is generator stream std::mt19937{seed + j} walked over the k inputs, the same
// stream the matvec operators use for output j with transpose=True, so that
// matmat(X)[i,:] == matvec(X[i,:], transpose=True) -- the identity the reference's tests assert
// (brainpylib/_src/jitconn_ops/tests/matmat_testcase.py:133-138).
//
// The reference kernel (lib/gpu_jitconn_matmat.cu:236-276) gives each thread a few rows of X for
// one column and reads X[row*k + id] with unrelated ids in neighbouring threads.  Here one
// wave64 owns a column: X is first transposed into a scratch buffer XT[k][m] (rows padded to a
// multiple of 64), then for every synapse (id, w) of the column the wave reads the contiguous
// row XT[id][0..m) and each lane accumulates its own output rows, in stream order, with the same
// multiply-then-add the CPU path performs.  The synapses of a batch pass from the lanes that drew
// them to the whole wave through LDS (one broadcast read each).
//
// Reference boundary: lib/gpu_jitconn_matmat.cu:279-317,364-455 (buffers = [X, Y], descriptor
// MatMatJITProbDescriptor1, target names lib/gpu_ops.cc:161-174).
#include "common.h"
#include "jitconn_stream.h"
#include "targets.h"

namespace bpl {
namespace {

constexpr int kTile = 32;

// XT[r / pass_rows][c][r % pass_rows] = X[r][c] for r < m: the transposed operand in slices of pass_rows rows of
// X (a multiple of 32), every slice contiguous, its rows pass_rows entries long; rows m .. m_pad - 1 are zero.
// (In one array of rows of m_pad entries the pieces that a pass reads lie m_pad entries apart and share a
// fraction of the L2's sets.)
template <typename T>
__global__ __launch_bounds__(kTile * 8) void transpose_pad_kernel(const T *__restrict__ X, T *__restrict__ XT,
                                                                  uint32_t m, uint32_t k, uint32_t m_pad,
                                                                  uint32_t pass_rows) {
  __shared__ T tile[kTile][kTile + 1];
  const uint32_t c0 = blockIdx.x * kTile, r0 = blockIdx.y * kTile;
  const uint32_t tx = threadIdx.x % kTile, ty = threadIdx.x / kTile;  // 32 x 8
  for (uint32_t i = ty; i < kTile; i += 8) {
    const uint32_t r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < m && c < k) ? X[static_cast<size_t>(r) * k + c] : T(0);
  }
  __syncthreads();
  for (uint32_t i = ty; i < kTile; i += 8) {
    const uint32_t c = c0 + i, r = r0 + tx;
    if (c < k && r < m_pad)
      XT[(static_cast<size_t>(r / pass_rows) * k + c) * pass_rows + r % pass_rows] = tile[tx][i];
  }
}

__device__ __forceinline__ float mul_rn(float a, float b) { return __fmul_rn(a, b); }
__device__ __forceinline__ double mul_rn(double a, double b) { return __dmul_rn(a, b); }
__device__ __forceinline__ float add_rn(float a, float b) { return __fadd_rn(a, b); }
__device__ __forceinline__ double add_rn(double a, double b) { return __dadd_rn(a, b); }

// one synapse of a batch: where its row of XT starts (bytes) and its weight
template <typename T1>
struct __attribute__((aligned(2 * sizeof(T1)))) Synapse {
  uint32_t off;
  T1 w;
};

// MT = 64-row tiles of Y one wave accumulates; a launch is one pass over MT * 64 rows of X (pass number `pass`).
// (The passes are launches of their own, one after the other: as the second dimension of one grid the
// workgroups of two passes run side by side nearly all the time, two slices of XT compete for the L2s, and
// eight passes of 256 rows took 5.7 ms instead of 3.8.)
template <typename T1, int W, int MT>
__global__ __launch_bounds__(256) void jitconn_matmat_kernel(const T1 *__restrict__ XT, T1 *__restrict__ Y,
                                                             uint32_t m, uint32_t k, uint32_t n, uint32_t m_pad,
                                                             uint32_t seed, double log_p, T1 wa, T1 wb,
                                                             uint32_t first, uint32_t count,
                                                             const uint32_t *__restrict__ states, uint32_t pass) {
  constexpr int kWaves = 4;
  constexpr int kWords = StreamLds<T1, W>::words;
  __shared__ __attribute__((aligned(8))) uint32_t s_state[kWaves * kWords];
  __shared__ Synapse<T1> s_syn[kWaves * kWave];
  const int lane = lane_id();
  const uint32_t wave = threadIdx.x / kWave;
  uint32_t *st = s_state + wave * kWords;
  Synapse<T1> *syn = s_syn + wave * kWave;
  const uint32_t row_base = pass * (MT * kWave);  // first row of Y of this pass
  // byte offsets into the pass's slice of XT fit 32 bits (checked by the host): one add per synapse instead of a
  // 64-bit product
  constexpr uint32_t row_bytes = MT * kWave * static_cast<uint32_t>(sizeof(T1));
  // (a wave-uniform base and a 32-bit offset per lane: one address add per synapse and the base in scalar registers)
  const char *xt_base = reinterpret_cast<const char *>(XT + static_cast<size_t>(pass) * k * (MT * kWave));
  const uint32_t lane_bytes = static_cast<uint32_t>(lane) * static_cast<uint32_t>(sizeof(T1));

  // columns first .. first + count - 1 of M, their generators seeded ahead: states[c] for column first + c
  for (uint32_t c = blockIdx.x * kWaves + wave; c < count; c += gridDim.x * kWaves) {
    const uint32_t j = first + c;
    T1 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = T1(0);
    const uint32_t *pre = states != nullptr ? states + static_cast<size_t>(c) * kMtN : nullptr;
    walk_stream<T1, W>(st, lane, seed + j, pre, k, log_p, wa, wb, [&](uint32_t idx, T1 w, bool valid) {
      // Every valid lane leaves its synapse (the byte offset of its row of XT, its weight) in the
      // wave's LDS slots, in lane order (which is stream order); every lane then reads the slots
      // one after the other (one address per read: a broadcast), so a synapse costs one LDS read,
      // one address add, MT loads and MT multiply-adds, with U synapses' loads in flight.
      const uint64_t mask = __ballot(valid);
      const uint32_t count = static_cast<uint32_t>(__popcll(mask));
      const uint32_t slot = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                                      __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
      __builtin_amdgcn_wave_barrier();  // the reads of the batch before are done
      if (valid) {
        syn[slot].off = idx * row_bytes;
        syn[slot].w = w;
      }
      __builtin_amdgcn_wave_barrier();
      constexpr int U = 8;
      uint32_t i = 0;
      for (; i + U <= count; i += U) {
        T1 ws[U];
        T1 x[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const Synapse<T1> e = syn[i + u];
          ws[u] = e.w;
          const T1 *row = reinterpret_cast<const T1 *>(xt_base + (e.off + lane_bytes));
#pragma unroll
          for (int t = 0; t < MT; ++t) x[u][t] = row[t * kWave];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int t = 0; t < MT; ++t) acc[t] = add_rn(acc[t], mul_rn(ws[u], x[u][t]));
        }
      }
      for (; i < count; ++i) {
        const Synapse<T1> e = syn[i];
        const T1 *row = reinterpret_cast<const T1 *>(xt_base + (e.off + lane_bytes));
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = add_rn(acc[t], mul_rn(e.w, row[t * kWave]));
      }
    });
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const uint32_t r = row_base + t * kWave + lane;
      if (r < m) Y[static_cast<size_t>(r) * n + j] = acc[t];
    }
  }
}

template <typename T1, int W>
void matmat_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t opaque_len) {
  bpl_matmat_jit_prob_descriptor d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (!(d.log_p < 0.0) || std::isinf(d.log_p)) {
    set_error("%s: log_p must be finite and negative (conn_prob in (0, 1]), got %g", target, d.log_p);
    return;
  }
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  const T1 *X = static_cast<const T1 *>(buffers[0]);
  T1 *Y = static_cast<T1 *>(buffers[1]);
  const uint32_t m = d.m, k = d.k, n = d.n;
  if (m == 0 || n == 0) return;
  // rows of X are padded to what the passes of the kernel read: one pass of 64 or 128 rows, or several of 128.
  // (A pass regenerates the matrix, but its slice of XT, 5 MB for 10,000 inputs, stays in the L2s: 2,048 rows of X
  // against a 10,000 x 10,000 matrix take 3.2 ms with uniform and 3.7 ms with normal weights in 16 passes of 128,
  // 3.7 and 3.8 ms in 8 passes of 256, whose slices do not.)
  uint32_t m_pad = (m + kWave - 1) / kWave * kWave;
  const uint32_t pass_rows = m_pad > 2 * kWave ? 2 * kWave : m_pad;
  m_pad = (m + pass_rows - 1) / pass_rows * pass_rows;
  if (k == 0) {
    fill_zero(stream, Y, m * n);  // m * n fits 32 bits whenever Y is addressable by the kernels below
    check_launch(target);
    return;
  }
  if (static_cast<uint64_t>(k) * pass_rows * sizeof(T1) > 0xffffffffull) {
    set_error("%s: a slice of the transposed operand (%u x %u) exceeds 4 GiB", target, k, pass_rows);
    return;
  }
  // scratch memory: [XT][the generator states of a chunk of columns, seeded ahead on the vector unit]
  const size_t xt_bytes = (static_cast<size_t>(k) * m_pad * sizeof(T1) + 255) / 256 * 256;
  // (from 32,768 columns on: with fewer a wave walks one or two columns and seeds them itself while others
  // compute: 10,000 columns 234 us, seeded ahead 259; 1,000,000 columns of 20 synapses 5.6 ms, seeded ahead 3.3)
  const bool ahead = n >= 32768;
  const uint32_t chunk = n < kSeedChunk ? n : kSeedChunk;
  const size_t state_bytes = ahead ? static_cast<size_t>(chunk) * kMtN * sizeof(uint32_t) : 0;
  unsigned char *ws = static_cast<unsigned char *>(stream_workspace(stream, xt_bytes + state_bytes));
  if (ws == nullptr) return;
  T1 *XT = reinterpret_cast<T1 *>(ws);
  uint32_t *states = reinterpret_cast<uint32_t *>(ws + xt_bytes);
  hipLaunchKernelGGL(transpose_pad_kernel<T1>, dim3(div_up(k, kTile), div_up(m_pad, kTile)), dim3(kTile * 8), 0,
                     stream, X, XT, m, k, m_pad, pass_rows);
  const T1 wa = static_cast<T1>(d.w_a), wb = static_cast<T1>(d.w_b);
  const uint32_t tiles = pass_rows / kWave, passes = m_pad / pass_rows;
  for (uint32_t first = 0; first < n; first += chunk) {
    const uint32_t count = n - first < chunk ? n - first : chunk;
    if (ahead) jitconn_seed_streams(stream, d.seed, first, count, states);
    const unsigned grid_x = div_up(count, 4);
    const uint32_t *pre = ahead ? states : nullptr;
    for (uint32_t pass = 0; pass < passes; ++pass) {
      if (tiles == 1) {
        hipLaunchKernelGGL((jitconn_matmat_kernel<T1, W, 1>), dim3(grid_x), dim3(256), 0, stream, XT, Y, m, k, n, m_pad,
                           d.seed, d.log_p, wa, wb, first, count, pre, pass);
      } else {
        hipLaunchKernelGGL((jitconn_matmat_kernel<T1, W, 2>), dim3(grid_x), dim3(256), 0, stream, XT, Y, m, k, n, m_pad,
                           d.seed, d.log_p, wa, wb, first, count, pre, pass);
      }
    }
  }
  check_launch(target);
}

}  // namespace
}  // namespace bpl

using namespace bpl;

#define BPL_DEFINE(name, T1, W)                                                                    \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    matmat_entry<T1, W>(__func__, static_cast<hipStream_t>(stream), buffers, opaque, opaque_len);   \
  }

BPL_DEFINE(gpu_matmat_prob_prob_normal_float_v1, float, kNormal)
BPL_DEFINE(gpu_matmat_prob_prob_normal_double_v1, double, kNormal)
BPL_DEFINE(gpu_matmat_prob_prob_uniform_float_v1, float, kUniform)
BPL_DEFINE(gpu_matmat_prob_prob_uniform_double_v1, double, kUniform)
