// coo_atomic_sum and coo_event_sum (lib/gpu_atomic_sum.cu, lib/gpu_event_sum.cu) for a long
// connection list and a result of a few windows: no atomics in memory.  Every workgroup takes a
// contiguous share of the connections and adds them into a window of the result in its LDS (weights:
// float64 accumulators; a homogeneous weight: 32-bit counts), the windows go to scratch memory, and
// a second kernel adds them in a fixed order: weights rounded once, a homogeneous weight as the sum
// of that many additions of it, which is what the reference's atomics leave whatever their order.
// A result wider than one window (16,384 float64 accumulators or 32,768 counts) is taken in slices by
// as many sets of workgroups, which all read the connections: two slices at most where a pass costs a
// gather per connection (weights, events), up to 32 where it reads the targets only (coo_atomic_sum
// with a homogeneous weight: 4 bytes per connection and slice).
// A wider result with a weight per connection or source goes through the coarse-sorted scatter of
// the CSR operators: bin_connections_kernel appends (position, weight) pairs to bins keyed by
// (producer, window of the result), sorted by window in LDS so that its stores merge, and
// add_uniform_bins adds every window's bins in float64 in LDS.  A homogeneous weight stays with counts
// (the sum of n additions of the weight is not n times the weight): slices, or the atomics.
// (One lane per connection with atomics on the result in memory: 1e8 connections 4.8 ms.)
#include <type_traits>

#include "bins.h"
#include "common.h"
#include "repeated_sum.h"
#include "window_sum.h"

namespace bpl {
namespace {

constexpr int kCooThreads = 1024;
constexpr size_t kCooWindowBytes = 128 * 1024;
template <bool HETER>
constexpr uint32_t coo_window_cols() { return static_cast<uint32_t>(kCooWindowBytes / (HETER ? sizeof(double) : sizeof(uint32_t))); }
template <bool HETER, bool EVENT>
constexpr uint32_t coo_max_slices() { return (HETER || EVENT) ? 2u : 32u; }
constexpr uint32_t kCooMinConnections = 1u << 17;  // below: the launch of a second kernel costs more than it saves

typedef uint32_t coo_u32x4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint64_t coo_u64x2 __attribute__((ext_vector_type(2), aligned(8)));
typedef float coo_f32x4 __attribute__((ext_vector_type(4), aligned(4)));
typedef double coo_f64x2 __attribute__((ext_vector_type(2), aligned(8)));

// four consecutive elements from an address that is a multiple of the element's size only; the lists pass
// through once (nontemporal)
__device__ __forceinline__ void load4(const uint32_t *p, uint64_t (&v)[4]) {
  const coo_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const coo_u32x4 *>(p));
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void load4(const uint64_t *p, uint64_t (&v)[4]) {
  const coo_u64x2 a = __builtin_nontemporal_load(reinterpret_cast<const coo_u64x2 *>(p));
  const coo_u64x2 b = __builtin_nontemporal_load(reinterpret_cast<const coo_u64x2 *>(p + 2));
  v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
}
__device__ __forceinline__ void load4(const float *p, float (&v)[4]) {
  const coo_f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const coo_f32x4 *>(p));
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void load4(const double *p, double (&v)[4]) {
  const coo_f64x2 a = __builtin_nontemporal_load(reinterpret_cast<const coo_f64x2 *>(p));
  const coo_f64x2 b = __builtin_nontemporal_load(reinterpret_cast<const coo_f64x2 *>(p + 2));
  v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
}

// grid = shares * slices; workgroup (share, slice) adds its share of the connections that fall into its slice
// of the result.  EVENT: connection i counts if events[pre_ids[i]] and carries values[i] (coo_event_sum);
// otherwise every connection counts and carries values[pre_ids[i]] (coo_atomic_sum).  A homogeneous
// weight (HETER false) is not read here: the window counts connections.  An id beyond the result is left out.
template <typename F, typename I, bool HETER, bool EVENT>
__global__ __launch_bounds__(kCooThreads) void coo_window_kernel(const uint8_t *__restrict__ events,
                                                                 const F *__restrict__ values,
                                                                 const I *__restrict__ post_ids,
                                                                 const I *__restrict__ pre_ids, uint32_t conn_size,
                                                                 uint32_t post_size, uint32_t slices,
                                                                 void *__restrict__ partial_raw) {
  using A = typename std::conditional<HETER, double, uint32_t>::type;
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  A *window = reinterpret_cast<A *>(smem_raw);
  const uint32_t tid = threadIdx.x;
  const uint32_t shares = gridDim.x / slices, share = blockIdx.x / slices, slice = blockIdx.x % slices;
  constexpr uint32_t kCols = coo_window_cols<HETER>();
  const uint32_t c_lo = slice * kCols;
  const uint32_t width = slices > 1 ? (post_size - c_lo < kCols ? post_size - c_lo : kCols) : post_size;
  for (uint32_t i = tid; i < width; i += kCooThreads) window[i] = A(0);
  __syncthreads();
  // shares of a multiple of 4 connections: a lane's four stay within one share
  const uint64_t per = ((static_cast<uint64_t>(conn_size) + shares - 1u) / shares + 3u) & ~3ull;
  const uint64_t a64 = static_cast<uint64_t>(share) * per, b64 = a64 + per;
  const uint32_t a = a64 < conn_size ? static_cast<uint32_t>(a64) : conn_size;
  const uint32_t b = b64 < conn_size ? static_cast<uint32_t>(b64) : conn_size;
  constexpr int U = 4, K = 2;  // a lane takes K groups of U consecutive connections per step
  for (uint64_t j0 = static_cast<uint64_t>(a) + U * tid; j0 < b; j0 += static_cast<uint64_t>(K) * U * kCooThreads) {
    uint64_t post[K][U], pre[K][U];
    F val[K][U];
    bool on[K][U];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const uint64_t j = j0 + static_cast<uint64_t>(k) * U * kCooThreads;
      if (j + U <= b) {
        load4(post_ids + j, post[k]);
        if (HETER || EVENT) load4(pre_ids + j, pre[k]);
        if (HETER && EVENT) load4(values + j, val[k]);
      } else {
#pragma unroll
        for (int t = 0; t < U; ++t) {
          const uint64_t jc = j + t < b ? j + t : b - 1u;
          post[k][t] = static_cast<uint64_t>(post_ids[jc]);
          if (HETER || EVENT) pre[k][t] = static_cast<uint64_t>(pre_ids[jc]);
          if (HETER && EVENT) val[k][t] = values[jc];
        }
      }
#pragma unroll
      for (int t = 0; t < U; ++t) on[k][t] = j + t < b;
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
      for (int t = 0; t < U; ++t) {
        if (EVENT) on[k][t] = on[k][t] && events[pre[k][t]] != 0;
        else if (HETER) val[k][t] = values[pre[k][t]];
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
      for (int t = 0; t < U; ++t) {
        const uint64_t rel = post[k][t] - c_lo;  // (wraps below c_lo)
        if (on[k][t] && rel < width) {
          if constexpr (HETER) atomicAdd(&window[rel], static_cast<double>(val[k][t]));
          else atomicAdd(&window[rel], 1u);
        }
      }
    }
  }
  __syncthreads();
  A *mine = static_cast<A *>(partial_raw) + static_cast<size_t>(share) * post_size + c_lo;
  for (uint32_t i = tid; i < width; i += kCooThreads) mine[i] = window[i];
}

template <typename F, bool HETER>
__global__ __launch_bounds__(kSumCols * kSumSlices) void coo_sum_windows_kernel(const void *__restrict__ partial,
                                                                                F *__restrict__ result,
                                                                                uint32_t post_size, uint32_t groups,
                                                                                const F *__restrict__ values) {
  using A = typename std::conditional<HETER, double, uint32_t>::type;
  using S = typename std::conditional<HETER, double, uint64_t>::type;
  bool mine;
  const S total = sum_windows_of_column<S, A>(static_cast<const A *>(partial), post_size, groups, &mine);
  if (mine) {
    const uint32_t c = blockIdx.x * kSumCols + threadIdx.x % kSumCols;
    if constexpr (HETER) result[c] = static_cast<F>(total);
    else result[c] = repeated_sum<F>(values[0], total);
  }
}

// ---- weights into a wide result: bins ----------------------------------------------------------
constexpr uint32_t kCooBinMinConnections = 1u << 20;
constexpr uint32_t kCooBinSlack = 128;           // pairs a bin holds beyond 5/4 of its even share
constexpr uint64_t kCooChunkBytes = 200ull << 20;  // pairs written and read back while they stay in the cache in
                                                  // front of the memory
constexpr uint32_t kCooWindowIdShift = 24;       // (positions within a window take kBinMaxShift bits, window ids 8)
static_assert(kBinMaxShift <= kCooWindowIdShift && kBinMaxWindows < (1u << (32 - kCooWindowIdShift)), "window id above the position");

// grid = producers; producer p takes an equal share of the connections [lo, hi) in rounds of 4,096: a lane
// loads four consecutive connections, ranks each within its window with an LDS counter, the round is
// sorted by window in LDS (offsets from a scan of the counters) and written out in that order to
// bin (p, w) = pairs + (p * n_win + w) * cap.  A pair that finds its bin full, and there are few (the bins hold
// 5/4 of an even spread), is added to the zeroed result with an atomic.  counts[w * producers + p]: pairs
// stored.  EVENT: connection i counts if events[pre_ids[i]] and carries values[i]; otherwise values[pre_ids[i]].
template <typename F, typename I, bool EVENT>
__global__ __launch_bounds__(kCooThreads) void bin_connections_kernel(
    const uint8_t *__restrict__ events, const F *__restrict__ values, const I *__restrict__ post_ids,
    const I *__restrict__ pre_ids, uint32_t lo, uint32_t hi, uint32_t post_size, F *__restrict__ result, uint32_t n_win,
    uint32_t shift, uint32_t cap, BinPair<F> *__restrict__ pairs, uint32_t *__restrict__ counts) {
  constexpr int U = 4;
  constexpr uint32_t kRound = U * kCooThreads;
  constexpr uint32_t kNone = kBinMaxWindows;  // window of a lane's slot that holds no pair
  __shared__ uint32_t s_cnt[kBinMaxWindows + 1];  // pairs of the current round, per window (and a spare counter)
  __shared__ uint32_t s_off[kBinMaxWindows + 1];  // their offsets in the sorted round, and the round's total
  __shared__ uint32_t s_total[kBinMaxWindows];    // pairs already in this producer's bins
  __shared__ uint32_t s_base[kBinMaxWindows];     // slot in the bin of the sorted round's pair i: s_base[window] + i
  __shared__ BinPair<F> s_sorted[kRound + 1];     // (and a spare slot; rel: the window's id above the position)
  const uint32_t tid = threadIdx.x, p = blockIdx.x, producers = gridDim.x;
  if (tid <= kBinMaxWindows) s_cnt[tid] = 0;
  if (tid < kBinMaxWindows) s_total[tid] = 0;
  const uint64_t per = ((static_cast<uint64_t>(hi - lo) + producers - 1u) / producers + 3u) & ~3ull;
  const uint64_t a64 = lo + static_cast<uint64_t>(p) * per, b64 = a64 + per;
  const uint32_t a = a64 < hi ? static_cast<uint32_t>(a64) : hi, b = b64 < hi ? static_cast<uint32_t>(b64) : hi;
  BinPair<F> *__restrict__ mine = pairs + static_cast<size_t>(p) * n_win * cap;
  __syncthreads();
  for (uint64_t base = a; base < b; base += kRound) {
    const uint64_t j = base + U * tid;
    uint64_t post[U], pre[U];
    F val[U];
    if (j + U <= b) {
      load4(post_ids + j, post);
      load4(pre_ids + j, pre);
      if (EVENT) load4(values + j, val);
    } else {
#pragma unroll
      for (int t = 0; t < U; ++t) {
        const uint64_t jc = j + t < b ? j + t : b - 1u;
        post[t] = static_cast<uint64_t>(post_ids[jc]);
        pre[t] = static_cast<uint64_t>(pre_ids[jc]);
        if (EVENT) val[t] = values[jc];
      }
    }
    uint32_t win[U], rel[U], rank[U];
#pragma unroll
    for (int t = 0; t < U; ++t) {
      bool on = j + t < b && post[t] < post_size;  // (an id beyond the result is left out)
      if (EVENT) on = on && events[pre[t]] != 0;
      else val[t] = values[pre[t]];
      win[t] = on ? static_cast<uint32_t>(post[t]) >> shift : kNone;
      rel[t] = static_cast<uint32_t>(post[t]) & ((1u << shift) - 1u);
    }
    // (only the lanes that hold a pair: with an event vector most hold none, and additions of many lanes to the
    // one spare counter would be taken one after the other, 64 cycles of the CU's LDS per instruction)
#pragma unroll
    for (int t = 0; t < U; ++t) {
      rank[t] = 0;
      if (win[t] != kNone) rank[t] = atomicAdd(&s_cnt[win[t]], 1u);
    }
    __syncthreads();
    if (tid < kWave) {  // offsets of the windows within the round: two counters per lane
      const uint32_t c0 = s_cnt[2 * tid], c1 = s_cnt[2 * tid + 1];
      const uint32_t incl = wave_inclusive_scan_u32(c0 + c1);
      const uint32_t o0 = incl - (c0 + c1), o1 = incl - c1;
      s_off[2 * tid] = o0;
      s_off[2 * tid + 1] = o1;
      if (tid == kWave - 1) s_off[kBinMaxWindows] = incl;
      const uint32_t t0 = s_total[2 * tid], t1 = s_total[2 * tid + 1];
      s_base[2 * tid] = t0 - o0;  // (modulo 2^32)
      s_base[2 * tid + 1] = t1 - o1;
      s_total[2 * tid] = t0 + c0;
      s_total[2 * tid + 1] = t1 + c1;
      s_cnt[2 * tid] = 0;
      s_cnt[2 * tid + 1] = 0;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < U; ++t) {
      BinPair<F> e;
      e.rel = rel[t] | (win[t] << kCooWindowIdShift);
      e.val = val[t];
      s_sorted[win[t] != kNone ? s_off[win[t]] + rank[t] : kRound] = e;
    }
    __syncthreads();
    // (No barrier behind the stores: the next round's counters are touched behind its first barrier only, its
    // sorted pairs behind its second.)
    const uint32_t round_total = s_off[kBinMaxWindows];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = tid + u * kCooThreads;
      if (i < round_total) {
        BinPair<F> e = s_sorted[i];
        const uint32_t w = e.rel >> kCooWindowIdShift;
        e.rel &= (1u << kCooWindowIdShift) - 1u;
        const uint32_t slot = s_base[w] + i;
        if (slot < cap) mine[static_cast<size_t>(w) * cap + slot] = e;
        else atomic_add(result + ((w << shift) | e.rel), e.val);
      }
    }
  }
  __syncthreads();
  if (tid < n_win) {
    const uint32_t c = s_total[tid];
    counts[static_cast<size_t>(tid) * producers + p] = c < cap ? c : cap;
  }
}

}  // namespace

template <bool HETER, bool EVENT>
bool coo_window_sum_usable(uint32_t conn_size, uint32_t post_size) {
  return conn_size >= kCooMinConnections && post_size != 0 &&
         post_size <= coo_max_slices<HETER, EVENT>() * coo_window_cols<HETER>();
}

// result (every element written) = the sum over the connections, as coo_window_kernel takes them.
// 1: enqueued.  0: nothing was enqueued, the caller takes its other path.  -1: nothing was enqueued and the
// call must fail, with the error that stands (the stream is being captured and the scratch memory would have
// to grow, or a launch failed).
template <typename F, typename I, bool HETER, bool EVENT>
int coo_window_sum(const char *target, hipStream_t stream, const uint8_t *events, const F *values, const I *post_ids,
                    const I *pre_ids, F *result, uint32_t conn_size, uint32_t post_size) {
  if (!coo_window_sum_usable<HETER, EVENT>(conn_size, post_size)) return 0;
  using A = typename std::conditional<HETER, double, uint32_t>::type;
  const uint32_t slices = div_up(post_size, coo_window_cols<HETER>());
  const size_t lds = static_cast<size_t>(slices > 1 ? coo_window_cols<HETER>() : post_size) * sizeof(A);
  auto kernel = coo_window_kernel<F, I, HETER, EVENT>;
  static thread_local bool attr_set = false;  // (one flag per instantiation)
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(kCooWindowBytes)) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    attr_set = true;
  }
  // two workgroups per CU where two windows fit its 160 KB of LDS; a share holds at least 16,384 connections
  const unsigned num_cu = static_cast<unsigned>(device_info().num_cu);
  unsigned shares = (lds <= 72 * 1024 ? 2u : 1u) * num_cu / slices;
  if (shares > conn_size / 16384u) shares = conn_size / 16384u;
  if (shares == 0) shares = 1;
  void *partial = stream_workspace(stream, static_cast<size_t>(shares) * post_size * sizeof(A));
  if (partial == nullptr) {
    if (scratch_refused_by_capture()) return -1;
    bpl_clear_error();  // (an allocation failed: the caller has its other path)
    return 0;
  }
  hipLaunchKernelGGL(kernel, dim3(shares * slices), dim3(kCooThreads), lds, stream, events, values, post_ids, pre_ids,
                     conn_size, post_size, slices, partial);
  hipLaunchKernelGGL((coo_sum_windows_kernel<F, HETER>), dim3(div_up(post_size, kSumCols)), dim3(kSumCols * kSumSlices), 0,
                     stream, static_cast<const void *>(partial), result, post_size, shares, values);
  return check_launch(target) ? 1 : -1;
}

// Weights into a result of more than two windows: bins.  Return values as coo_window_sum.
template <typename F, typename I, bool EVENT>
int coo_bin_sum(const char *target, hipStream_t stream, const uint8_t *events, const F *values, const I *post_ids,
                const I *pre_ids, F *result, uint32_t conn_size, uint32_t post_size) {
  if (conn_size < kCooBinMinConnections || post_size == 0) return 0;
  const uint32_t shift = bin_window_shift(post_size);
  const uint32_t n_win = div_up(post_size, 1u << shift);
  if (n_win < 2 || n_win > kBinMaxWindows) return 0;
  const uint32_t producers = 2u * static_cast<uint32_t>(device_info().num_cu);
  uint32_t chunks = div_up(static_cast<uint64_t>(conn_size) * sizeof(BinPair<F>), kCooChunkBytes);
  if (chunks == 0) chunks = 1;
  const uint32_t chunk_conn = (div_up(conn_size, chunks) + 3u) & ~3u;
  const uint32_t per = (div_up(chunk_conn, producers) + 3u) & ~3u;  // as the kernel divides a whole chunk
  const uint32_t even = per / n_win;
  const uint32_t cap = (even + even / 4u + kCooBinSlack + 3u) & ~3u;
  const size_t pair_bytes = (static_cast<size_t>(producers) * n_win * cap * sizeof(BinPair<F>) + 255) / 256 * 256;
  const size_t count_bytes = static_cast<size_t>(n_win) * producers * sizeof(uint32_t);
  unsigned char *ws = static_cast<unsigned char *>(stream_workspace(stream, pair_bytes + count_bytes));
  if (ws == nullptr) {
    if (scratch_refused_by_capture()) return -1;
    bpl_clear_error();  // (an allocation failed: the caller has its other path)
    return 0;
  }
  BinPair<F> *pairs = reinterpret_cast<BinPair<F> *>(ws);
  uint32_t *counts = reinterpret_cast<uint32_t *>(ws + pair_bytes);
  fill_zero(stream, result, post_size);
  for (uint64_t lo = 0; lo < conn_size; lo += chunk_conn) {
    const uint32_t hi = lo + chunk_conn < conn_size ? static_cast<uint32_t>(lo + chunk_conn) : conn_size;
    hipLaunchKernelGGL((bin_connections_kernel<F, I, EVENT>), dim3(producers), dim3(kCooThreads), 0, stream, events, values,
                       post_ids, pre_ids, static_cast<uint32_t>(lo), hi, post_size, result, n_win, shift, cap, pairs, counts);
    if (!add_uniform_bins<F>(target, stream, result, post_size, shift, producers, cap, pairs, false, counts, nullptr)) return -1;
  }
  return check_launch(target) ? 1 : -1;
}

#define BPL_COO_WINDOW_SUM(F, I)                                                                                       \
  template int coo_window_sum<F, I, false, false>(const char *, hipStream_t, const uint8_t *, const F *, const I *,  \
                                                   const I *, F *, uint32_t, uint32_t);                                \
  template int coo_window_sum<F, I, true, false>(const char *, hipStream_t, const uint8_t *, const F *, const I *,   \
                                                  const I *, F *, uint32_t, uint32_t);                                 \
  template int coo_window_sum<F, I, false, true>(const char *, hipStream_t, const uint8_t *, const F *, const I *,   \
                                                  const I *, F *, uint32_t, uint32_t);                                 \
  template int coo_window_sum<F, I, true, true>(const char *, hipStream_t, const uint8_t *, const F *, const I *,    \
                                                 const I *, F *, uint32_t, uint32_t);                                  \
  template int coo_bin_sum<F, I, false>(const char *, hipStream_t, const uint8_t *, const F *, const I *, const I *,  \
                                        F *, uint32_t, uint32_t);                                                      \
  template int coo_bin_sum<F, I, true>(const char *, hipStream_t, const uint8_t *, const F *, const I *, const I *,   \
                                       F *, uint32_t, uint32_t);
BPL_COO_WINDOW_SUM(float, uint32_t)
BPL_COO_WINDOW_SUM(float, uint64_t)
BPL_COO_WINDOW_SUM(double, uint32_t)
BPL_COO_WINDOW_SUM(double, uint64_t)
#undef BPL_COO_WINDOW_SUM

}  // namespace bpl
