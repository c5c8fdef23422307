// event_csr_matvec and csr_matvec for gfx950 (wave64).
//
// Two kernel families serve both operators:
//
//   scatter  (transpose):  y[indices[j]] += w(j)  for the nonzeros j of the rows r that are "on"
//            A workgroup owns 64 consecutive rows.  Wave 0 tests the rows' events, compacts the
//            active rows and prefix-sums their lengths in LDS (ballot + DPP scan); then all 256
//            threads walk the workgroup's active nonzeros as ONE flat range, so lanes stay
//            coalesced along a row and the load per thread is even whatever the mix of active
//            and silent rows.  Additions are hardware fp32/fp64 atomics in L2.
//
//   gather   (no transpose):  y[r] = sum_j w(j) * x(indices[j])
//            Persistent workgroups stream the rows; G lanes cooperate on one row (G = 64, 32,
//            16 or 8, picked on the device from the mean row length, which the host does not
//            know).  For event vectors the workgroup first packs the events into an LDS bitmap,
//            so the per-nonzero test is an LDS bit probe instead of a random global byte load,
//            and `data` is only fetched where the probe hits.  Per-lane partial sums are kept
//            in fp64 and rounded once, like the reference CPU path's `r = 0.` accumulator
//            (brainpylib/_src/event_ops/event_csr_matvec.py:342-347,
//             brainpylib/_src/sparse_ops/sparse_csr_matvec.py:116-119).
//
// Reference boundary: lib/gpu_event_csr_matvec.cu:148-260, lib/gpu_csr_matvec.cu:84-135,195-246,
// 505-621 (buffer order, descriptor, target names).
#include <mutex>
#include <type_traits>

#include "common.h"
#include "csr_flat_gather.h"
#include "repeated_sum.h"
#include "targets.h"

namespace bpl {
namespace {

constexpr int kScatterRows = 64;     // rows owned by one scatter workgroup

// The host does not know the number of nonzeros (it is indptr[n_row], in device memory), so where
// the better kernel depends on the mean row length both candidates are launched and each one
// returns at once unless the count lies in its range.
struct NnzGate {
  uint32_t lo, hi;  // run iff lo <= indptr[n_row] <= hi
  __device__ __forceinline__ bool open(const uint32_t *__restrict__ indptr, uint32_t n_row) const {
    if (lo == 0 && hi == 0xffffffffu) return true;
    const uint32_t nnz = indptr[n_row];
    return nnz >= lo && nnz <= hi;
  }
};
constexpr NnzGate kAlways = {0u, 0xffffffffu};
constexpr int kScatterThreads = 256;

enum : int { kEvent = 0, kDense = 1 };

// A homogeneous weight delivered by n synapses.  The reference adds the weight once per synapse:
// in place in the precision of the output when it scatters (event_csr_matvec.py:313-331), into a
// float64 accumulator that is rounded once when it gathers (event_csr_matvec.py:334-357).  Every
// addend being the same, the result depends on the count alone, so kernels that count in integers
// reproduce the reference's bits whatever order the synapses arrive in.
template <typename F>
__device__ __forceinline__ F scattered_sum(F w, uint64_t n) {
  return repeated_sum<F>(w, n);
}
__device__ __forceinline__ float gathered_sum(float w, uint32_t n) {
  // up to 2^29 additions of a 24-bit weight are exact in float64: the product, rounded once.  The sum starts
  // from +0: a weight of -0 (or no synapse at all) leaves +0, as 0 + (-0) does
  return static_cast<float>(0.0 + static_cast<double>(w) * static_cast<double>(n));
}
__device__ __forceinline__ double gathered_sum(double w, uint32_t n) { return repeated_sum<double>(w, n); }

// A synapse count kept in the storage of an output element until the last kernel of a call turns
// it into the sum (float: the 32 bits hold the integer; double: the count as a number, exact).
__device__ __forceinline__ float count_as_element(uint32_t n, float) { return __uint_as_float(n); }
__device__ __forceinline__ double count_as_element(uint32_t n, double) { return static_cast<double>(n); }
__device__ __forceinline__ uint64_t element_as_count(float v) { return __float_as_uint(v); }
__device__ __forceinline__ uint64_t element_as_count(double v) { return static_cast<uint64_t>(v); }
// adds n to the count held in *y (y zeroed before)
__device__ __forceinline__ void add_count(float *y, uint32_t n) { atomicAdd(reinterpret_cast<uint32_t *>(y), n); }
__device__ __forceinline__ void add_count(double *y, uint32_t n) {
  // (the count as a number: float64 atomic adds of integers are exact and commute)
  atomic_add(y, static_cast<double>(n));
}

// y[i] = the sum of y[i]'s count of synapses of weight data[0] (see above), in place
template <typename F>
__global__ __launch_bounds__(256) void counts_to_sums_kernel(F *__restrict__ y, uint32_t n, const F *__restrict__ data,
                                                             const uint32_t *__restrict__ indptr, uint32_t n_row,
                                                             NnzGate gate) {
  if (!gate.open(indptr, n_row)) return;
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < n) y[i] = scattered_sum<F>(data[0], element_as_count(y[i]));
}

// ------------------------------------------------------------------------------------------------
// scatter
// ------------------------------------------------------------------------------------------------
template <typename F, typename VT, bool HETER, int MODE>
__global__ __launch_bounds__(kScatterThreads) void csr_scatter_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const VT *__restrict__ x, F *__restrict__ y, uint32_t n_row, NnzGate gate) {
  if (!gate.open(indptr, n_row)) return;
  __shared__ uint32_t s_start[kScatterRows];  // first nonzero of the k-th active row
  __shared__ uint32_t s_off[kScatterRows];    // position of that row in the flat range
  __shared__ F s_scale[kScatterRows];         // dense mode: x[r]
  __shared__ uint32_t s_count, s_total;

  const uint32_t tid = threadIdx.x;
  if (tid < kWave) {
    const uint32_t r = blockIdx.x * kScatterRows + tid;
    bool on = false;
    uint32_t start = 0, len = 0;
    F scale = F(1);
    if (r < n_row) {
      if (MODE == kEvent) {
        on = is_event(x[r]);
      } else {
        scale = static_cast<F>(x[r]);
        on = true;
      }
      if (on) {
        start = indptr[r];
        len = indptr[r + 1] - start;
        on = len != 0;
      }
    }
    if (!on) len = 0;
    const uint64_t mask = __ballot(on);
    const uint32_t incl = wave_inclusive_scan_u32(len);
    const int pos = __popcll(mask & ((1ull << tid) - 1ull));
    if (on) {
      s_start[pos] = start;
      s_off[pos] = incl - len;
      if (MODE == kDense) s_scale[pos] = scale;
    }
    if (tid == kWave - 1) {
      s_count = static_cast<uint32_t>(__popcll(mask));
      s_total = incl;
    }
  }
  __syncthreads();
  const uint32_t count = s_count;
  const uint32_t total = s_total;
  if (count == 0) return;

  const F w_homo = HETER ? F(0) : data[0];

  constexpr int U = 4;
  for (uint32_t e0 = tid; e0 < total; e0 += U * kScatterThreads) {
    uint32_t j[U];
    uint32_t col[U];
    F w[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t e = e0 + u * kScatterThreads;
      ok[u] = e < total;
      // largest k < count with s_off[k] <= e
      uint32_t k = 0;
#pragma unroll
      for (uint32_t step = kScatterRows / 2; step > 0; step >>= 1) {
        const uint32_t mid = k + step;
        if (mid < count && s_off[mid] <= e) k = mid;
      }
      j[u] = s_start[k] + (e - s_off[k]);
      w[u] = (MODE == kDense) ? s_scale[k] : F(1);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) {
        col[u] = indices[j[u]];
        const F d = HETER ? data[j[u]] : w_homo;
        // dense: v * values[j] (heter) or values * v (homo), as the reference CPU loop multiplies
        w[u] = (MODE == kDense) ? static_cast<F>(w[u] * d) : d;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) atomic_add(&y[col[u]], w[u]);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// scatter, output window in LDS
// ------------------------------------------------------------------------------------------------
// Random global atomics retire at about one cache-line request per lane; the same additions made
// in LDS and written out once, lane-contiguous, need a small fraction of the requests.  When
// the output vector can be cut into a few windows that fit in LDS, workgroup (g, b) owns row
// group g and output window b: it compacts the group's active rows, streams their column
// indices (every window's workgroup reads them; they come from L2 / Infinity Cache after the
// first), fetches `data` only for the nonzeros that fall into its window, accumulates them with
// LDS atomics and finally adds the window's nonzero entries to y with contiguous atomics.
constexpr int kWinThreads = 1024;
constexpr int kWinMaxRows = 2048;  // rows per workgroup = capacity of the active-row list

// Active rows of the whole matrix, gathered once into a list in device memory (any order):
// (first nonzero, length) per row whose input is nonzero and that has nonzeros, plus the input
// value in dense mode.  The kernels that follow take equal shares of the LIST, so their work does
// not depend on where in the matrix the activity is.  A workgroup tests 1,024 rows per unit of
// kCollectPerThread and reserves its list positions with one atomic (atomics on one address
// retire at about 15 ns each, whoever issues them: one per 1,024 rows cost 14 us for a million rows).
// Optional chores for the kernels that follow: `clear[0 .. n_clear)` and `zero[0 .. n_zero)` are set to zero.
// I: the type of the row offsets.  64-bit offsets (the older csr_event_sum) are listed as 32-bit (first
// nonzero, length) too; a matrix of 2^32 nonzeros or more is not listed at all (the chores are still done
// and the list stays empty: the caller has a kernel for such matrices that runs in that case only).
template <typename F, typename VT, int MODE, int kCollectPerThread, typename I = uint32_t>
__global__ __launch_bounds__(kWinThreads) void collect_active_rows_kernel(
    const I *__restrict__ indptr, const VT *__restrict__ x, uint32_t n_row, uint32_t *__restrict__ counter,
    uint2 *__restrict__ list, F *__restrict__ scales, NnzGate gate, uint32_t *__restrict__ clear, uint32_t n_clear,
    F *__restrict__ zero, uint32_t n_zero) {
  // (The list holds n_row entries.  The counter is zero when a call starts, so positions stay below
  // n_row; should an earlier call have failed half way and left it set, nothing is written beyond.)
  if constexpr (sizeof(I) == 4) {
    if (!gate.open(reinterpret_cast<const uint32_t *>(indptr), n_row)) return;
  }
  __shared__ uint32_t s_count, s_base;
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  if (tid == 0) s_count = 0;
  for (uint32_t i = blockIdx.x * kWinThreads + tid; i < n_clear; i += gridDim.x * kWinThreads) clear[i] = 0u;
  for (uint32_t i = blockIdx.x * kWinThreads + tid; i < n_zero; i += gridDim.x * kWinThreads) zero[i] = F(0);
  if constexpr (sizeof(I) == 8) {
    if ((static_cast<uint64_t>(indptr[n_row]) >> 32) != 0) return;
  }
  __syncthreads();
  const uint32_t r0 = blockIdx.x * (kWinThreads * kCollectPerThread) + tid;
  bool on[kCollectPerThread];
  uint32_t start[kCollectPerThread], len[kCollectPerThread], at[kCollectPerThread];
  F scale[kCollectPerThread];
#pragma unroll
  for (int e = 0; e < kCollectPerThread; ++e) {
    const uint32_t r = r0 + e * kWinThreads;
    on[e] = false;
    scale[e] = F(1);
    if (r < n_row) {
      if (MODE == kEvent) {
        on[e] = is_event(x[r]);
      } else {
        scale[e] = static_cast<F>(x[r]);
        on[e] = true;  // also a zero input: 0 * inf and 0 * NaN must reach the output (cusparse_matvec.py:204-211)
      }
    }
  }
#pragma unroll
  for (int e = 0; e < kCollectPerThread; ++e) {
    start[e] = len[e] = at[e] = 0;
    if (on[e]) {
      const uint32_t r = r0 + e * kWinThreads;
      start[e] = static_cast<uint32_t>(indptr[r]);
      len[e] = static_cast<uint32_t>(indptr[r + 1]) - start[e];
      on[e] = len[e] != 0;
    }
  }
#pragma unroll
  for (int e = 0; e < kCollectPerThread; ++e) {
    const uint64_t mask = __ballot(on[e]);
    uint32_t base = 0;
    if (lane == 0 && mask) base = atomicAdd(&s_count, static_cast<uint32_t>(__popcll(mask)));
    base = __builtin_amdgcn_readfirstlane(base);
    at[e] = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
  }
  __syncthreads();
  if (tid == 0) s_base = s_count ? atomicAdd(counter, s_count) : 0u;
  __syncthreads();
  const uint32_t base = s_base;
#pragma unroll
  for (int e = 0; e < kCollectPerThread; ++e) {
    if (on[e] && base + at[e] < n_row) {
      list[base + at[e]] = make_uint2(start[e], len[e]);
      if (MODE == kDense) scales[base + at[e]] = scale[e];
    }
  }
}

template <typename F, typename VT, int MODE>
unsigned collect_workgroups(uint32_t n_row) {
  return n_row > 262144u ? div_up(n_row, 4 * kWinThreads) : div_up(n_row, kWinThreads);
}
template <typename F, typename VT, int MODE, typename I = uint32_t>
void launch_collect(hipStream_t stream, const I *indptr, const VT *x, uint32_t n_row, uint32_t *counter,
                    uint2 *list, F *scales, NnzGate gate, uint32_t *clear, uint32_t n_clear, F *zero, uint32_t n_zero) {
  const unsigned wgs = collect_workgroups<F, VT, MODE>(n_row);
  if (n_row > 262144u)
    hipLaunchKernelGGL((collect_active_rows_kernel<F, VT, MODE, 4, I>), dim3(wgs), dim3(kWinThreads), 0, stream, indptr, x,
                       n_row, counter, list, scales, gate, clear, n_clear, zero, n_zero);
  else
    hipLaunchKernelGGL((collect_active_rows_kernel<F, VT, MODE, 1, I>), dim3(wgs), dim3(kWinThreads), 0, stream, indptr, x,
                       n_row, counter, list, scales, gate, clear, n_clear, zero, n_zero);
}

// The same list over the rows of every entry of a batch of event vectors that share one matrix:
// virtual row v = entry * n_row + r; `colbase` receives entry * n_col for every listed row.
// events: [events_batch][n_row]; entry bi of this launch is entry first_entry + bi of the whole
// batch and reads row (first_entry + bi) % events_batch.
template <typename F, typename VT>
__global__ __launch_bounds__(kWinThreads) void collect_active_rows_batched_kernel(
    const uint32_t *__restrict__ indptr, const VT *__restrict__ events, uint32_t n_row, uint32_t n_col,
    uint32_t batch, uint32_t events_batch, uint32_t first_entry, uint32_t *__restrict__ counter,
    uint2 *__restrict__ list,
    uint32_t *__restrict__ colbase, uint32_t *__restrict__ clear, uint32_t n_clear, F *__restrict__ zero,
    uint64_t n_zero) {
  constexpr int kPer = 8;
  __shared__ uint32_t s_count, s_base;
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  if (tid == 0) s_count = 0;
  for (uint32_t i = blockIdx.x * kWinThreads + tid; i < n_clear; i += gridDim.x * kWinThreads) clear[i] = 0u;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kWinThreads + tid; i < n_zero;
       i += static_cast<uint64_t>(gridDim.x) * kWinThreads)
    zero[i] = F(0);
  __syncthreads();
  const uint64_t total = static_cast<uint64_t>(batch) * n_row;
  const uint64_t v0 = static_cast<uint64_t>(blockIdx.x) * (kWinThreads * kPer) + tid;
  bool on[kPer];
  uint32_t start[kPer], len[kPer], at[kPer], base_col[kPer];
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const uint64_t v = v0 + static_cast<uint64_t>(e) * kWinThreads;
    on[e] = false;
    start[e] = len[e] = at[e] = base_col[e] = 0;
    if (v < total) {
      const uint32_t bi = static_cast<uint32_t>(v / n_row), r = static_cast<uint32_t>(v % n_row);
      on[e] = is_event(events[static_cast<size_t>((first_entry + bi) % events_batch) * n_row + r]);
      if (on[e]) {
        start[e] = indptr[r];
        len[e] = indptr[r + 1] - start[e];
        on[e] = len[e] != 0;
        base_col[e] = bi * n_col;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const uint64_t mask = __ballot(on[e]);
    uint32_t base = 0;
    if (lane == 0 && mask) base = atomicAdd(&s_count, static_cast<uint32_t>(__popcll(mask)));
    base = __builtin_amdgcn_readfirstlane(base);
    at[e] = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
  }
  __syncthreads();
  if (tid == 0) s_base = s_count ? atomicAdd(counter, s_count) : 0u;
  __syncthreads();
  const uint32_t base = s_base;
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    if (on[e] && base + at[e] < total) {  // (the list holds batch * n_row entries)
      list[base + at[e]] = make_uint2(start[e], len[e]);
      colbase[base + at[e]] = base_col[e];
    }
  }
}

// Row groups that take part in a launch whose active rows are listed in device memory: one per
// 32,768 active nonzeros (estimated from the mean row length) or per 128 active rows (a wave walks
// its rows one after the other, a memory round trip or two each: short rows are bound by their
// number), at least one, at most the launched number.  Every group writes a slice of partial outputs
// that the summing kernel reads again, so with little activity a few groups finish sooner than a
// chip full of them.
__device__ __forceinline__ uint32_t groups_in_use(uint32_t active_rows, uint32_t nnz, uint32_t n_row,
                                                 uint32_t launched) {
  const uint64_t work = static_cast<uint64_t>(active_rows) * (nnz / n_row + 1u);
  const uint64_t by_work = (work + 32767u) / 32768u, by_rows = (active_rows + 127u) / 128u;
  const uint64_t want = by_work > by_rows ? by_work : by_rows;
  return want < 1u ? 1u : want > launched ? launched : static_cast<uint32_t>(want);
}

// A = type of the window's accumulators: F, or double where every lane adds (dense input):
// 64-bit LDS float adds retire nine times faster than 32-bit ones on this device.
template <typename F, typename VT, bool HETER, int MODE, typename A>
__global__ __launch_bounds__(kWinThreads) void csr_scatter_window_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const VT *__restrict__ x, F *__restrict__ y, uint32_t n_row, uint32_t n_col, uint32_t rows_per_wg,
    uint32_t win, uint32_t n_win, F *__restrict__ partial, NnzGate gate,
    uint32_t *__restrict__ active_count, const uint2 *__restrict__ active_list,
    const F *__restrict__ active_scales) {
  if (!gate.open(indptr, n_row)) return;
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  // (Measured on this device: the LDS unit adds 32-bit floats at about a third of a lane per clock
  // and CU, 64-bit floats nine times and 32-bit integers thirty times faster.  For sparse event
  // input a float64 window would halve the window and double the passes over the indices, which
  // costs what the faster additions save at the sizes tried: A = F there.)
  // With a homogeneous weight and event input the window counts synapses instead (32-bit integer
  // LDS adds, exact) and the weight is multiplied in once per output at the end.
  constexpr bool kCount = !HETER && MODE == kEvent;
  A *window = reinterpret_cast<A *>(smem_raw);
  uint32_t *cwindow = reinterpret_cast<uint32_t *>(smem_raw);
  F *s_scale = reinterpret_cast<F *>(window + win);  // dense mode: x[r] per active row
  uint32_t *s_start = reinterpret_cast<uint32_t *>(s_scale + (MODE == kDense ? kWinMaxRows : 0));
  uint32_t *s_len = s_start + kWinMaxRows;
  __shared__ uint32_t s_count, s_next;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid % kWave, wave = tid / kWave;
  constexpr uint32_t kWaves = kWinThreads / kWave;
  // Workgroups are dealt to the 8 XCDs round robin by blockIdx.  The n_win workgroups of one row
  // group read the same index and weight runs, so they are renumbered to sit on one XCD and
  // share its L2: ids [x * per_xcd, (x + 1) * per_xcd) belong to XCD x.
  uint32_t id = blockIdx.x;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t per_xcd = gridDim.x / kXcds;
    if (id < per_xcd * kXcds) id = (id % kXcds) * per_xcd + id / kXcds;
  }
  const uint32_t b = id % n_win;
  uint32_t g = id / n_win;
  // With a device list only the first groups_in_use() groups work, in an order that deals
  // consecutive groups to different XCDs; the choice goes to the summing kernel through the
  // stream's second counter.
  uint32_t groups = gridDim.x / n_win;
  if (active_list != nullptr) {
    const uint32_t launched = groups;
    if (launched % 8u == 0) g = (g % (launched / 8u)) * 8u + g / (launched / 8u);
    groups = groups_in_use(active_count[0] < n_row ? active_count[0] : n_row, indptr[n_row], n_row, launched);
    if (g == 0 && b == 0 && threadIdx.x == 0) active_count[1] = groups;
    if (g >= groups) return;
  }
  const uint32_t c0 = b * win;
  const uint32_t width = (c0 + win <= n_col) ? win : n_col - c0;

  const F w_homo = HETER ? F(0) : data[0];
  for (uint32_t i = tid; i < width; i += kWinThreads) {
    if (kCount) cwindow[i] = 0u;
    else window[i] = A(0);
  }

  // Source of the active rows: this group's share of the list made by collect_active_rows_kernel,
  // or (active_list == nullptr) the group's own rows_per_wg rows, tested here.  Either way they are
  // taken kWinMaxRows at a time, the capacity of the list in LDS.
  uint32_t span_lo = 0, span_hi = rows_per_wg;
  if (active_list != nullptr) {
    const uint32_t total = active_count[0] < n_row ? active_count[0] : n_row;  // (the list's capacity)
    span_lo = static_cast<uint32_t>(static_cast<uint64_t>(g) * total / groups);
    span_hi = static_cast<uint32_t>(static_cast<uint64_t>(g + 1) * total / groups);
  }
  for (uint32_t chunk0 = span_lo; chunk0 < span_hi; chunk0 += kWinMaxRows) {
  const uint32_t chunk_rows = (span_hi - chunk0 < kWinMaxRows) ? span_hi - chunk0 : kWinMaxRows;
  if (active_list == nullptr && static_cast<uint64_t>(g) * rows_per_wg + chunk0 >= n_row) break;  // uniform
  if (tid == 0) s_count = (active_list != nullptr) ? chunk_rows : 0u, s_next = kWaves;
  __syncthreads();

  if (active_list != nullptr) {
    for (uint32_t i = tid; i < chunk_rows; i += kWinThreads) {
      const uint2 e = active_list[chunk0 + i];
      s_start[i] = e.x;
      s_len[i] = e.y;
      if (MODE == kDense) s_scale[i] = active_scales[chunk0 + i];
    }
  }
  // else: active rows of the chunk, tested here (order does not matter)
  for (uint32_t t0 = 0; active_list == nullptr && t0 < chunk_rows; t0 += kWinThreads) {
    const uint32_t r = g * rows_per_wg + chunk0 + t0 + tid;
    bool on = false;
    uint32_t start = 0, len = 0;
    F scale = F(1);
    if (t0 + tid < chunk_rows && r < n_row) {
      if (MODE == kEvent) {
        on = is_event(x[r]);
      } else {
        scale = static_cast<F>(x[r]);
        on = true;  // also a zero input, whose products with inf and NaN weights are NaN
      }
      if (on) {
        start = indptr[r];
        len = indptr[r + 1] - start;
        on = len != 0;
      }
    }
    const uint64_t mask = __ballot(on);
    uint32_t base = 0;
    if (lane == 0 && mask) base = atomicAdd(&s_count, static_cast<uint32_t>(__popcll(mask)));
    base = __builtin_amdgcn_readfirstlane(base);
    if (on) {
      const uint32_t k = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
      s_start[k] = start;
      s_len[k] = len;
      if (MODE == kDense) s_scale[k] = scale;
    }
  }
  __syncthreads();
  const uint32_t count = s_count;

  // Waves take active rows from a shared counter and walk them in steps of U*64 nonzeros.  The
  // column indices of the next step (of this row or of the next row taken) are requested
  // before this step's weights are loaded and added, so that the two latencies overlap.
  constexpr int U = 8;
  auto load_rel = [&](const uint32_t *ip, uint32_t b0, uint32_t len, uint32_t (&rel)[U]) {
    if (b0 + U * kWave <= len) {
#pragma unroll
      for (int u = 0; u < U; ++u) rel[u] = ip[b0 + u * kWave + lane] - c0;
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t j = b0 + u * kWave + lane;
        rel[u] = 0xffffffffu;  // outside every window
        if (j < len) rel[u] = ip[j] - c0;
      }
    }
  };
  uint32_t k = wave;
  uint32_t start = 0, len = 0, b0 = 0;
  F scale = F(1);
  uint32_t rel[U];
  if (k < count) {
    start = s_start[k], len = s_len[k];
    if (MODE == kDense) scale = s_scale[k];
    load_rel(indices + start, 0, len, rel);
  }
  while (k < count) {
    // where the next step is
    uint32_t nk = k, nstart = start, nlen = len, nb0 = b0 + U * kWave;
    F nscale = scale;
    if (nb0 >= len) {
      uint32_t t = 0;
      if (lane == 0) t = atomicAdd(&s_next, 1u);
      nk = __builtin_amdgcn_readfirstlane(t);
      nb0 = 0;
      if (nk < count) {
        nstart = s_start[nk], nlen = s_len[nk];
        if (MODE == kDense) nscale = s_scale[nk];
      }
    }
    uint32_t nrel[U];
    if (nk < count) load_rel(indices + nstart, nb0, nlen, nrel);
    // this step: all weight loads first, then the LDS atomics
    const F *dp = data + (HETER ? start : 0u);
    F w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      w[u] = w_homo;
      if (HETER && rel[u] < width) w[u] = dp[b0 + u * kWave + lane];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (rel[u] < width) {
        if (kCount) atomicAdd(&cwindow[rel[u]], 1u);
        else atomicAdd(&window[rel[u]], static_cast<A>((MODE == kDense) ? static_cast<F>(scale * w[u]) : w[u]));
      }
    }
    k = nk, start = nstart, len = nlen, b0 = nb0, scale = nscale;
#pragma unroll
    for (int u = 0; u < U; ++u) rel[u] = nrel[u];
  }
  __syncthreads();  // the lists and counters are reused by the next chunk; the window is complete after the last
  }

  if (partial != nullptr) {
    // plain contiguous stores of the whole window into this row group's slice; a second
    // kernel sums the slices
    // (counting windows leave their counts: the summing kernel adds the integers and forms the sum once)
    F *dst = partial + static_cast<size_t>(g) * n_col + c0;
    for (uint32_t i = tid; i < width; i += kWinThreads) {
      if constexpr (kCount) dst[i] = count_as_element(cwindow[i], F(0));
      else dst[i] = static_cast<F>(window[i]);
    }
  } else if constexpr (kCount) {
    // counts into the zeroed y; counts_to_sums_kernel follows
    for (uint32_t i = tid; i < width; i += kWinThreads)
      if (cwindow[i] != 0u) add_count(&y[c0 + i], cwindow[i]);
  } else {
    for (uint32_t i = tid; i < width; i += kWinThreads) {
      const F v = static_cast<F>(window[i]);
      if (v != F(0)) atomic_add(&y[c0 + i], v);
    }
  }
}

// y[c] = sum over row groups of partial[g][c]
// (COUNT: the slices hold synapse counts of the homogeneous weight data[0])
template <typename F, bool COUNT>
__global__ __launch_bounds__(256) void sum_partials_kernel(const F *__restrict__ partial, F *__restrict__ y,
                                                           uint32_t n_col, uint32_t groups,
                                                           const uint32_t *__restrict__ indptr, uint32_t n_row,
                                                           NnzGate gate, uint32_t *__restrict__ reset,
                                                           const F *__restrict__ data) {
  if (!gate.open(indptr, n_row)) return;
  // with a device list of active rows: the groups that took part, as the window kernel left them
  // in the second counter; the active-row counter itself goes back to zero for the next call
  if (reset != nullptr) {
    groups = reset[1];
    if (blockIdx.x == 0 && threadIdx.x == 0) reset[0] = 0u;
  }
  const uint32_t c = blockIdx.x * 256u + threadIdx.x;
  if (c >= n_col) return;
  if constexpr (COUNT) {
    uint64_t n = 0;
    for (uint32_t g = 0; g < groups; ++g) n += element_as_count(partial[static_cast<size_t>(g) * n_col + c]);
    y[c] = scattered_sum<F>(data[0], n);
    return;
  }
  F acc = F(0);
  uint32_t g = 0;
  for (; g + 16 <= groups; g += 16) {  // (sixteen loads in flight: with hundreds of groups a column is a chain of round trips)
    F a[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) a[k] = partial[static_cast<size_t>(g + k) * n_col + c];
#pragma unroll
    for (int k = 0; k < 16; k += 4) acc += (a[k] + a[k + 1]) + (a[k + 2] + a[k + 3]);
  }
  for (; g + 4 <= groups; g += 4) {
    const F a0 = partial[static_cast<size_t>(g) * n_col + c];
    const F a1 = partial[static_cast<size_t>(g + 1) * n_col + c];
    const F a2 = partial[static_cast<size_t>(g + 2) * n_col + c];
    const F a3 = partial[static_cast<size_t>(g + 3) * n_col + c];
    acc += (a0 + a1) + (a2 + a3);
  }
  for (; g < groups; ++g) acc += partial[static_cast<size_t>(g) * n_col + c];
  y[c] = acc;
}

// ------------------------------------------------------------------------------------------------
// gather
// ------------------------------------------------------------------------------------------------

constexpr uint32_t kHubSteps = 64;  // a row of more steps than this is left to the whole workgroup (gather_hub_rows)

// G lanes walk the rows assigned to their group as ONE sequence of steps of U*G nonzeros: the
// column indices of the next step (which may belong to the group's next row) are requested
// before the loads that depend on the current step's indices are consumed, so a row change
// does not drain the pipeline.  Loads are unconditional (out-of-row lanes re-read a valid
// element and are masked out of the sum); only the `data` fetch of an event hit is predicated.
// Is column `col` an event?  BITS 0: the event vector in global memory; 1, 2: the bitmap in LDS;
// 3: a coarse bitmap in LDS (one bit per 2^g columns), then the exact packed one in global memory.
template <int BITS, typename VT>
__device__ __forceinline__ bool event_hit(const uint32_t *s_bits, const VT *__restrict__ x, uint32_t col, uint32_t g) {
  if constexpr (BITS == 0) {
    return probe_event(x, col);
  } else if constexpr (BITS == 3) {
    const uint32_t c = col >> g;
    return ((s_bits[c >> 5] >> (c & 31u)) & 1u) && probe_event(x, col);
  } else {
    return (s_bits[col >> 5] >> (col & 31u)) & 1u;
  }
}

// The same for the U columns of a step.  With the two-level bitmap the loads of the exact words are
// issued for all U columns before any is looked at (lanes whose coarse bit is clear read word 0),
// so that they are in flight together instead of one behind the other.
template <int BITS, int U, typename VT>
__device__ __forceinline__ void event_hits(const uint32_t *s_bits, const VT *__restrict__ x, const uint32_t (&col)[U],
                                           uint32_t g, bool (&hit)[U]) {
  if constexpr (BITS == 3) {
    uint32_t word[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t c = col[u] >> g;
      hit[u] = (s_bits[c >> 5] >> (c & 31u)) & 1u;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) word[u] = x[hit[u] ? col[u] >> 5 : 0u].w;
#pragma unroll
    for (int u = 0; u < U; ++u) hit[u] = hit[u] && ((word[u] >> (col[u] & 31u)) & 1u);
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) hit[u] = event_hit<BITS>(s_bits, x, col[u], g);
  }
}

// Element `col` of the dense vector.  BITS == 2: its first `lds_n` elements are staged in LDS
// (`s_x`), the rest is gathered from global memory.
template <typename VT, int BITS>
__device__ __forceinline__ VT dense_element(const VT *__restrict__ x, const uint32_t *s_x, uint32_t lds_n, uint32_t col) {
  if constexpr (BITS == 2) {
    if (col < lds_n) return reinterpret_cast<const VT *>(s_x)[col];
  }
  return x[col];
}

typedef uint32_t row_u32x4 __attribute__((ext_vector_type(4), aligned(4)));  // (a row begins at any nonzero)
typedef float row_f32x4 __attribute__((ext_vector_type(4), aligned(4)));
template <typename F, typename VT, bool HETER, int MODE, int BITS, int G, int U>
__device__ __forceinline__ void gather_rows(const F *__restrict__ data, const uint32_t *__restrict__ indices,
                                            const uint32_t *__restrict__ indptr, const VT *__restrict__ x,
                                            F *__restrict__ y, uint32_t n_row, const uint32_t *s_bits,
                                            uint32_t coarse_g) {
  const uint32_t groups_per_block = blockDim.x / G;
  const uint32_t gl = threadIdx.x % G;
  const uint32_t total_groups = gridDim.x * groups_per_block;
  const F w_homo = HETER ? F(0) : data[0];
  // A lane takes its U nonzeros of a step as U / Q runs of Q consecutive ones, each with ONE load of Q indices
  // (and weights): slot u of lane gl is nonzero Q * ((u / Q) * G + gl) + u % Q of the step.  With a nonzero per
  // load a group's G lanes asked for G * 4 bytes of a line per instruction and for the same line again with the
  // next one, U times over.
  // (not with the dense vector staged in LDS, float: that walk has no registers to spare for two workgroups per CU)
  constexpr int Q = ((U == 4 || U == 8) && !(MODE == kDense && BITS == 1)) ? 4 : 1;
  auto slot = [&](int u) { return static_cast<uint32_t>(Q * ((u / Q) * G) + u % Q) + static_cast<uint32_t>(Q) * gl; };
  const uint32_t nnz = Q > 1 ? indptr[n_row] : 0u;  // (a run of Q is loaded whole only where the arrays hold all of it)
  // A row of more than kHubSteps steps looks empty here: gather_hub_rows() gives it to the whole workgroup.
  constexpr uint32_t hub_len = kHubSteps * U * G;
  auto bounds = [&](uint32_t r, uint32_t &s, uint32_t &e) {
    s = indptr[r], e = indptr[r + 1];
    if (e - s > hub_len) e = s;
  };

  uint32_t row = blockIdx.x * groups_per_block + threadIdx.x / G;
  if (row >= n_row) return;
  uint32_t base, end;                                         // current step: [base, base + U*G) of this row
  bounds(row, base, end);
  uint32_t nrow_start = 0, nrow_end = 0;                      // bounds of the group's next row
  if (row + total_groups < n_row) bounds(row + total_groups, nrow_start, nrow_end);

  auto load_cols = [&](uint32_t b, uint32_t e, uint32_t (&c)[U]) {
    const uint32_t safe = e ? e - 1 : 0u;  // any valid element (the matrix has at least one)
    if constexpr (Q > 1) {
      if (static_cast<uint64_t>(b) + U * G <= nnz) {
        // (what lies beyond the row's end are the next rows' indices: valid columns, left out by their number)
#pragma unroll
        for (int q = 0; q < U / Q; ++q) {
          const row_u32x4 v = *reinterpret_cast<const row_u32x4 *>(indices + b + slot(Q * q));
          c[Q * q] = v.x, c[Q * q + 1] = v.y, c[Q * q + 2] = v.z, c[Q * q + 3] = v.w;
        }
        return;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = b + slot(u);
      c[u] = indices[j < e ? j : safe];
    }
  };
  auto load_weights = [&](uint32_t b, uint32_t e, auto &d) {  // (dense vector: every weight of the step)
    if constexpr (Q > 1 && sizeof(F) == 4) {
      if (static_cast<uint64_t>(b) + U * G <= nnz) {
#pragma unroll
        for (int q = 0; q < U / Q; ++q) {
          const row_f32x4 v = *reinterpret_cast<const row_f32x4 *>(data + b + slot(Q * q));
          d[Q * q] = v.x, d[Q * q + 1] = v.y, d[Q * q + 2] = v.z, d[Q * q + 3] = v.w;
        }
        return;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = b + slot(u);
      d[u] = data[j < e ? j : (e ? e - 1 : 0u)];
    }
  };

  uint32_t col[U];
  load_cols(base, end, col);
  double acc = 0.0;   // heter / dense
  uint32_t hits = 0;  // homo event: number of active synapses
  while (true) {
    // where the next step is
    const bool last_of_row = base + U * G >= end;
    const uint32_t next_row = last_of_row ? row + total_groups : row;
    const uint32_t next_base = last_of_row ? nrow_start : base + U * G;
    const uint32_t next_end = last_of_row ? nrow_end : end;
    const bool more = next_row < n_row;

    // loads that depend on this step's indices
    F val[U];
    bool use[U];
    bool hits_u[U];
    // (sixteen weights in registers beside sixteen columns are more than two workgroups per CU leave room for)
    constexpr bool kWeightRuns = MODE == kDense && HETER && Q > 1;
    F wgt[kWeightRuns ? U : 1];
    if constexpr (kWeightRuns) load_weights(base, end, wgt);
    if constexpr (MODE == kEvent && BITS == 3) event_hits<BITS, U>(s_bits, x, col, coarse_g, hits_u);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = base + slot(u);
      const bool ok = j < end;
      if (MODE == kEvent) {
        bool hit;
        if constexpr (BITS == 3) hit = hits_u[u];
        else hit = event_hit<BITS>(s_bits, x, col[u], coarse_g);
        hit = hit && ok;
        use[u] = hit;
        val[u] = F(0);
        if (HETER && hit) val[u] = data[j];
      } else {
        use[u] = ok;
        F d = w_homo;
        if constexpr (kWeightRuns) d = wgt[u];
        else if constexpr (HETER) d = data[ok ? j : (end ? end - 1 : 0u)];
        // product formed in F, then widened (the reference multiplies two F values)
        val[u] = static_cast<F>(static_cast<F>(dense_element<VT, BITS>(x, s_bits, coarse_g, col[u])) * d);
      }
    }
    // indices of the next step, and the row bounds one row further ahead
    uint32_t coln[U];
    if (more) {
      load_cols(next_base, next_end, coln);
      if (last_of_row && next_row + total_groups < n_row) bounds(next_row + total_groups, nrow_start, nrow_end);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (MODE == kEvent && !HETER) hits += use[u] ? 1u : 0u;
      else acc += use[u] ? static_cast<double>(val[u]) : 0.0;
    }
    if (last_of_row) {
      if (MODE == kEvent && !HETER) {
        hits = group_sum<G>(hits);
        // n additions of the same fp32 value into a float64 accumulator are exact: n * w
        if (gl == 0) y[row] = gathered_sum(w_homo, hits);
        hits = 0;
      } else {
        acc = group_sum<G>(acc);
        if (gl == 0) y[row] = static_cast<F>(acc);
        acc = 0.0;
      }
    }
    if (!more) break;
    row = next_row, base = next_base, end = next_end;
#pragma unroll
    for (int u = 0; u < U; ++u) col[u] = coln[u];
  }
}

// An index or weight of a long row: the arrays pass through once and a wave's load instruction covers whole
// lines, so the load is marked nontemporal (the event gather of 1e8 nonzeros in rows of 1,000: 124 -> 115 us
// at 5 % events, 92 -> 82 us at 1 %).  Not for the short rows above, where a few lanes take a piece of a
// line per instruction and the line is wanted again by the next: 2,000,000 rows of 30 took 182 instead of 118 us.
template <typename T>
__device__ __forceinline__ T stream_load(const T *p) { return __builtin_nontemporal_load(p); }

// Long rows: one wave per row.  Row bounds and base pointers are wave uniform (scalar
// registers), lanes address their elements as base + small offset, full steps of U*64 nonzeros
// run without guards and only the last step of a row is predicated.
template <typename F, typename VT, bool HETER, int MODE, int BITS, int U>
__device__ __forceinline__ void gather_rows_wave(const F *__restrict__ data, const uint32_t *__restrict__ indices,
                                                 const uint32_t *__restrict__ indptr, const VT *__restrict__ x,
                                                 F *__restrict__ y, uint32_t n_row, const uint32_t *s_bits,
                                                 uint32_t coarse_g) {
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const uint32_t waves_per_block = blockDim.x / kWave;
  const uint32_t total_waves = gridDim.x * waves_per_block;
  const F w_homo = HETER ? F(0) : data[0];

  auto step = [&](const uint32_t *ip, const F *dp, uint32_t b, uint32_t len, bool guard, double &acc, uint32_t &hits) {
    uint32_t col[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t off = b + u * kWave + lane;
      ok[u] = !guard || off < len;
      // (heterogeneous weights: lanes past the end of the row re-read its last index, a plain load that
      // is masked out of the sum; 3 % faster there than a predicated load, 2 % slower with one weight)
      if (HETER) col[u] = stream_load(ip + (ok[u] ? off : len - 1u));
      else col[u] = ok[u] ? stream_load(ip + off) : 0u;
    }
    F val[U];
    bool hits_u[U];
    if constexpr (MODE == kEvent && BITS == 3) event_hits<BITS, U>(s_bits, x, col, coarse_g, hits_u);  // (col 0 where !ok)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t off = b + u * kWave + lane;
      if (MODE == kEvent) {
        bool hit;
        if constexpr (BITS == 3) hit = hits_u[u];
        else if (BITS == 1 || BITS == 2) hit = event_hit<BITS>(s_bits, x, col[u], coarse_g);
        else hit = ok[u] && event_hit<BITS>(s_bits, x, col[u], coarse_g);
        hit = hit && ok[u];
        if (HETER) {
          val[u] = F(0);
          if (hit) val[u] = stream_load(dp + off);
        } else {
          hits += hit ? 1u : 0u;
        }
      } else {
        val[u] = F(0);
        if (ok[u]) {
          const F d = HETER ? stream_load(dp + off) : w_homo;
          // product formed in F, then widened (the reference multiplies two F values)
          val[u] = static_cast<F>(static_cast<F>(dense_element<VT, BITS>(x, s_bits, coarse_g, col[u])) * d);
        }
      }
    }
    if (!(MODE == kEvent && !HETER)) {
#pragma unroll
      for (int u = 0; u < U; ++u) acc += static_cast<double>(val[u]);
    }
  };

  for (uint32_t row = blockIdx.x * waves_per_block + threadIdx.x / kWave; row < n_row; row += total_waves) {
    const uint32_t urow = __builtin_amdgcn_readfirstlane(row);
    const uint32_t start = indptr[urow];
    const uint32_t len = indptr[urow + 1] - start;
    if (len > kHubSteps * U * kWave) continue;  // (a whole workgroup takes it and stores it: gather_hub_rows())
    const uint32_t *ip = indices + start;
    const F *dp = data + (HETER ? start : 0u);
    double acc = 0.0;
    uint32_t hits = 0;
    // Rows that lie a multiple of 4 KB apart (1,024 nonzeros each, say) would have every wave of the device at the
    // same offset within 4 KB at the same time, and with it on the same memory channels (1,024 per row: 16 % slower
    // per nonzero than 1,000 per row).  So the rows begin at different full steps, by their number, and wrap.
    const uint32_t full = len / (U * kWave);  // steps without a guard
    const uint32_t first = urow & (full >= 4u ? 3u : full >= 2u ? 1u : 0u);
    for (uint32_t i = first; i < full; ++i) step(ip, dp, i * (U * kWave), len, false, acc, hits);
    for (uint32_t i = 0; i < first; ++i) step(ip, dp, i * (U * kWave), len, false, acc, hits);
    if (full * (U * kWave) < len) step(ip, dp, full * (U * kWave), len, true, acc, hits);
    if (MODE == kEvent && !HETER) {
      hits = wave_sum(hits);
      // n additions of the same fp32 value into a float64 accumulator are exact: n * w
      if (lane == 0) y[urow] = gathered_sum(w_homo, hits);
    } else {
      acc = wave_sum(acc);
      if (lane == 0) y[urow] = static_cast<F>(acc);
    }
  }
}

// Hub rows.  The walks above give a row to G lanes (or one wave), so one row that holds a large share
// of the nonzeros would be walked by a handful of lanes while the rest of the device is done (a row of
// 1e6 nonzeros among 20,000 of 50: 19 ms).  They treat a row of more than kHubSteps of their steps as
// empty, and after its walk every workgroup looks through the bounds of the rows it was dealt again
// (workgroup b: rows b * gpb + g + k * total_groups, g < gpb) and walks each such row with all its
// threads: partial sums per lane, a wave sum, one float64 (or integer) LDS atomic per wave.
// The walk with a wave per row skips such rows without storing anything, and they are dealt one by one
// (gpb = 1: workgroup b looks at rows b, b + gridDim.x, ...): in a matrix of a few thousand rows that are
// all this long, sixteen consecutive rows per workgroup would leave most of the device idle (2,000 rows of
// 50,000: an eighth of the workgroups had rows).
template <typename F, typename VT, bool HETER, int MODE, int BITS>
__device__ __forceinline__ void gather_hub_rows(const F *__restrict__ data, const uint32_t *__restrict__ indices,
                                                const uint32_t *__restrict__ indptr, const VT *__restrict__ x,
                                                F *__restrict__ y, uint32_t n_row, const uint32_t *s_bits,
                                                uint32_t coarse_g, uint32_t gpb, uint32_t hub_len) {
  __shared__ unsigned long long s_mask[1024 / kWave];
  __shared__ double s_acc;
  __shared__ uint32_t s_hits;
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave, nwaves = blockDim.x / kWave;
  const uint32_t total_groups = gridDim.x * gpb;
  const uint32_t first = blockIdx.x * gpb;
  if (first >= n_row) return;
  const uint32_t count = ((n_row - first + total_groups - 1u) / total_groups) * gpb;  // rows dealt to this workgroup
  const F w_homo = HETER ? F(0) : data[0];
  auto row_of = [&](uint32_t i) { return (i / gpb) * total_groups + first + (i % gpb); };
  for (uint32_t i0 = 0; i0 < count; i0 += blockDim.x) {
    bool hub = false;
    if (i0 + tid < count) {
      const uint32_t r = row_of(i0 + tid);
      if (r < n_row) hub = indptr[r + 1] - indptr[r] > hub_len;
    }
    const unsigned long long mine = __ballot(hub);
    if (!__syncthreads_or(hub)) continue;  // (the usual case: none)
    if (lane == 0) s_mask[wave] = mine;
    __syncthreads();
    for (uint32_t w = 0; w < nwaves; ++w) {
      unsigned long long m = s_mask[w];
      while (m != 0) {
        const uint32_t r = row_of(i0 + w * kWave + static_cast<uint32_t>(__ffsll(m) - 1));
        m &= m - 1ull;
        if (tid == 0) s_acc = 0.0, s_hits = 0u;
        __syncthreads();
        const uint32_t start = indptr[r], len = indptr[r + 1] - start;
        double acc = 0.0;
        uint32_t hits = 0;
        constexpr uint32_t U = 4;  // loads in flight per lane and step; the next step's are requested before this one's are used
        uint32_t col[U], ncol[U];
        auto load_cols = [&](uint32_t j0, uint32_t (&c)[U]) {  // (beyond the row: its last index again)
#pragma unroll
          for (uint32_t u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * blockDim.x;
            c[u] = indices[start + (j < len ? j : len - 1u)];
          }
        };
        load_cols(tid, col);
        for (uint32_t j0 = tid; j0 < len; j0 += U * blockDim.x) {
          load_cols(j0 + U * blockDim.x, ncol);
#pragma unroll
          for (uint32_t u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * blockDim.x;
            if (j >= len) continue;
            if (MODE == kEvent) {
              if (event_hit<BITS>(s_bits, x, col[u], coarse_g)) {
                if (HETER) acc += static_cast<double>(data[start + j]);
                else ++hits;
              }
            } else {
              const F d = HETER ? data[start + j] : w_homo;
              acc += static_cast<double>(static_cast<F>(static_cast<F>(dense_element<VT, BITS>(x, s_bits, coarse_g, col[u])) * d));
            }
          }
#pragma unroll
          for (uint32_t u = 0; u < U; ++u) col[u] = ncol[u];
        }
        if (MODE == kEvent && !HETER) {
          hits = wave_sum(hits);
          if (lane == 0 && hits != 0u) atomicAdd(&s_hits, hits);
        } else {
          acc = wave_sum(acc);
          if (lane == 0) atomicAdd(&s_acc, acc);
        }
        __syncthreads();
        if (tid == 0) y[r] = (MODE == kEvent && !HETER) ? gathered_sum(w_homo, s_hits) : static_cast<F>(s_acc);
        __syncthreads();
      }
    }
  }
}


// ------------------------------------------------------------------------------------------------
// event gather, walked flat (rows of 16 to 383 nonzeros on average)
// ------------------------------------------------------------------------------------------------
// The row-wise walks pad every row to whole steps of its lane group: with 100 nonzeros per row and 8 lanes
// x 16 loads per row a quarter of the index requests lie beyond their row.  Here every wave owns a contiguous
// range of the nonzeros that begins and ends at row boundaries (the rows whose first nonzero lies in its
// equal share of the nonzeros: no row is shared by two waves, so nothing is left for a second kernel) and
// takes it in steps of 768 or 1,280: three or five 16-byte nontemporal loads of indices per lane (the next
// step's are under way while a step is worked on), twelve or twenty probes of the event bitmap in LDS per
// lane.  Rows are looked up for the HITS only: the lanes leave the positions of their hits (some 5 % of the
// nonzeros) in a queue in LDS, compacted by a prefix sum over the wave, and every lane then takes one hit: its
// weight, a six-step search of a window of 65 row offsets in LDS for its row, one atomic addition to that
// row's accumulator (float64; a homogeneous weight: a 32-bit count).  Rows that end inside the step are stored.
constexpr uint32_t kFlatEvRows = 64;     // rows of a window (one per lane)
constexpr uint32_t kFlatEvMinMean = 16, kFlatEvMaxMean = 384;
constexpr uint32_t kFlatEvSharedMaxMean = 256, kFlatEvSharedMinNnz = 45000000;  // (in the kernel that shares its CU)
constexpr uint32_t kFlatEvWaves = 16;
// Loads of four indices per lane and step, and sets of index registers (steps under way).  One workgroup per CU (a
// bitmap of more than 80 KB): 5 and 2 (steps of 1,280 nonzeros; measured against 3..8 loads and 2 or 3 sets: 4 and 3
// took 146 / 94 us for 1,000,000 x 1,000,000 with 100 per row, weights per nonzero / one weight, 5 and 2 141 / 86; steps
// that are a power of two in bytes were the slowest of their neighbours every time).  Two workgroups per CU must keep to
// 64 registers: 3 and 2.
constexpr int kFlatEvQuadsAlone = 5, kFlatEvDepthAlone = 2, kFlatEvQuadsShared = 3, kFlatEvDepthShared = 2;
// hits queued at a time (more in a step: further rounds)
constexpr uint32_t kFlatEvQueueAlone = 256, kFlatEvQueueShared = 128;
// LDS of the walk behind the bitmap: accumulators, windows of row offsets and queues of 16 waves
constexpr size_t flat_event_wave_bytes(uint32_t queue) { return kFlatEvRows * 8 + (kFlatEvRows + 4) * 4 + queue * 2; }
constexpr size_t flat_event_lds_bytes(uint32_t queue) { return kFlatEvWaves * flat_event_wave_bytes(queue); }
// the largest event bitmap that is kept whole in LDS (beside that; wider event vectors get a two-level bitmap)
constexpr size_t kLdsEventBitmapCap = (kLdsBitmapCap - flat_event_lds_bytes(kFlatEvQueueAlone)) / 256 * 256;
// the largest bitmap that leaves room for two workgroups per CU (80 KB each, less the kernel's static LDS)
constexpr size_t kLdsSharedBitmapCap = 80 * 1024 - 512;
// where the walk's memory begins behind a bitmap of n_col bits (in 32-bit words)
__host__ __device__ inline uint32_t flat_event_lds_offset(uint32_t n_col) { return ((n_col + 31u) / 32u + 3u) & ~3u; }
// Whether a workgroup of the kernel that shares its CU is given the walk's memory behind its bitmap (the
// launcher and the kernel decide alike)
__host__ __device__ inline bool flat_event_shared_fits(uint32_t n_row, uint32_t n_col) {
  return n_row >= 16384u &&
         static_cast<size_t>(flat_event_lds_offset(n_col)) * 4 + flat_event_lds_bytes(kFlatEvQueueShared) <= kLdsSharedBitmapCap;
}

// For each of two positions pos <= indptr[n_row]: the first row r in [0, n_row] with indptr[r] >= pos.  The wave
// searches together, 64 probes a round, and both searches go round by round side by side (their probes are
// under way together: half the dependent round trips of one search after the other).
__device__ __forceinline__ void first_rows_from(const uint32_t *__restrict__ indptr, uint32_t n_row, uint32_t pos_a,
                                                uint32_t pos_b, uint32_t lane, uint32_t &row_a, uint32_t &row_b) {
  // an answer lies in [lo, hi]: indptr[r] < pos for r < lo, indptr[hi] >= pos
  uint32_t lo_a = 0, hi_a = n_row, lo_b = 0, hi_b = n_row;
  while (lo_a < hi_a || lo_b < hi_b) {
    const uint32_t span_a = hi_a - lo_a, span_b = hi_b - lo_b;
    const uint32_t stride_a = span_a / kWave + (span_a % kWave ? 1u : 0u);
    const uint32_t stride_b = span_b / kWave + (span_b % kWave ? 1u : 0u);
    const uint64_t probe_a = static_cast<uint64_t>(lo_a) + static_cast<uint64_t>(lane) * stride_a;
    const uint64_t probe_b = static_cast<uint64_t>(lo_b) + static_cast<uint64_t>(lane) * stride_b;
    const uint32_t at_a = probe_a < hi_a ? indptr[probe_a] : 0xffffffffu;
    const uint32_t at_b = probe_b < hi_b ? indptr[probe_b] : 0xffffffffu;
    // (the lanes whose probe lies below the position form a prefix)
    const uint32_t cnt_a = static_cast<uint32_t>(__popcll(__ballot(probe_a < hi_a && at_a < pos_a)));
    const uint32_t cnt_b = static_cast<uint32_t>(__popcll(__ballot(probe_b < hi_b && at_b < pos_b)));
    if (cnt_a == 0) {
      hi_a = lo_a;  // indptr[lo] >= pos
    } else {
      // indptr[lo + (cnt - 1) stride] < pos, and the probe after it (if it lies below hi) is not below pos
      const uint64_t next = static_cast<uint64_t>(lo_a) + static_cast<uint64_t>(cnt_a) * stride_a;
      if (next < hi_a) hi_a = static_cast<uint32_t>(next);
      lo_a += (cnt_a - 1u) * stride_a + 1u;
    }
    if (cnt_b == 0) {
      hi_b = lo_b;
    } else {
      const uint64_t next = static_cast<uint64_t>(lo_b) + static_cast<uint64_t>(cnt_b) * stride_b;
      if (next < hi_b) hi_b = static_cast<uint32_t>(next);
      lo_b += (cnt_b - 1u) * stride_b + 1u;
    }
  }
  row_a = lo_a;
  row_b = lo_b;
}

template <typename F, bool HETER, int U, int DEPTH, uint32_t QUEUE>
__device__ __forceinline__ void gather_rows_flat_event(const F *__restrict__ data, const uint32_t *__restrict__ indices,
                                                       const uint32_t *__restrict__ indptr, F *__restrict__ y,
                                                       uint32_t n_row, uint32_t nnz, const uint32_t *s_bits,
                                                       uint32_t *s_work) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  using A = typename std::conditional<HETER, double, uint32_t>::type;
  static_assert(DEPTH == 2 || DEPTH == 3, "two or three sets of index registers");
  constexpr uint32_t kStep = 4u * U * kWave;  // nonzeros per step
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wv = threadIdx.x / kWave;
  // the wave's part of `s_work` (16-byte aligned): 64 accumulators, 66 row offsets, the queue
  uint32_t *mine_lds = s_work + wv * (flat_event_wave_bytes(QUEUE) / 4);
  A *s_sum = reinterpret_cast<A *>(mine_lds);
  uint32_t *s_ptr = mine_lds + kFlatEvRows * 2;
  uint16_t *s_queue = reinterpret_cast<uint16_t *>(s_ptr + kFlatEvRows + 4);
  const uint32_t waves = gridDim.x * (blockDim.x / kWave), w = blockIdx.x * (blockDim.x / kWave) + wv;
  const F w_homo = HETER ? F(0) : data[0];
  // equal shares of the nonzeros, in whole steps; the wave's rows are those that begin in its share
  const uint64_t share = ((static_cast<uint64_t>(nnz) + waves - 1u) / waves + kStep - 1u) / kStep * kStep;
  const uint64_t pos0 = static_cast<uint64_t>(w) * share, pos1 = pos0 + share;
  if (pos0 >= nnz) return;  // (nnz > 0, so wave 0 goes on)
  uint32_t r, r_last;
  first_rows_from(indptr, n_row, static_cast<uint32_t>(pos0), pos1 >= nnz ? nnz : static_cast<uint32_t>(pos1), lane, r, r_last);
  const uint32_t r_end = (pos1 >= nnz) ? n_row : r_last;  // (the last wave also takes the rows without nonzeros at the end)
  if (r >= r_end) return;
  const uint32_t begin = indptr[r], end = indptr[r_end];
  if (begin == end) {  // rows without nonzeros only
    for (uint32_t i = r + lane; i < r_end; i += kWave) y[i] = F(0);
    return;
  }
  s_sum[lane] = A(0);
  if (lane == 0) s_ptr[kFlatEvRows + 1] = 0xffffffffu;

  // the step that begins at nonzero s0: lane l takes the quads s0 / 4 + l, + 64, ...
  // Every lane loads, without a condition: a quad beyond the array's last whole one is replaced by that one (its
  // hits are masked below, in the last step of a range, and the array's last, partial quad is probed there).
  const uint32_t q_last = nnz / 4u - 1u;
  auto load_indices = [&](uint32_t s0, u32x4 (&ci)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t q = s0 / 4u + static_cast<uint32_t>(u) * kWave + lane;
      ci[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(indices) + (q < q_last ? q : q_last));
    }
  };
  // the window of row offsets from row r on
  uint32_t ptr_lane, ptr_last;
  auto load_window = [&]() {
    const uint64_t k = static_cast<uint64_t>(r) + lane;
    ptr_lane = k <= n_row ? indptr[k] : 0xffffffffu;
    ptr_last = static_cast<uint64_t>(r) + kFlatEvRows <= n_row ? indptr[r + kFlatEvRows] : 0xffffffffu;
  };
  auto store_window = [&]() {
    s_ptr[lane] = ptr_lane;
    if (lane == 0) s_ptr[kFlatEvRows] = ptr_last;
  };
  // The indices of the next DEPTH - 1 steps are under way while a step is worked on (with one step ahead and 16
  // waves per CU the walk streamed at 3.4 TB/s).  Every step works from a set of registers of its own and, at its
  // END, requests the step DEPTH ahead into the same set (copying between sets would wait for the request just
  // made); the request comes behind the gathers of the hits' weights, because waiting for a load means waiting
  // for every load issued before it.  The window of row offsets of the next step is requested just before.
  // (The first requests are made in the order in which the steps make them, and kept in that order: how many
  // later requests a wait may leave under way is fixed at compile time from BOTH ways into the loop.)
  u32x4 ci0[U], ci1[U], ci2[DEPTH == 3 ? U : 1];
  const uint32_t first_step = begin / 4u * 4u;  // (steps begin at whole quads; what lies before `begin` is masked)
  load_window();
  __builtin_amdgcn_sched_barrier(0);
  load_indices(first_step, ci0);
  __builtin_amdgcn_sched_barrier(0);
  load_indices(first_step + kStep, ci1);
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (DEPTH == 3) load_indices(first_step + 2u * kStep, ci2);
  __builtin_amdgcn_sched_barrier(0);
  auto step = [&](const uint32_t s0, u32x4 (&ci)[U]) {
    const uint32_t s1 = (end - s0 > kStep) ? s0 + kStep : end;
    // the probes: bit 4 u + t of `hits` = nonzero s0 + 256 u + 4 lane + t is in the range and its column has an event
    uint32_t hits = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t c[4] = {ci[u].x, ci[u].y, ci[u].z, ci[u].w};
#pragma unroll
      for (int t = 0; t < 4; ++t)  // (the bit-field extract takes the low five bits of its offset)
        hits |= __builtin_amdgcn_ubfe(s_bits[c[t] >> 5], c[t], 1u) << (4 * u + t);
    }
    if (s0 < begin || s1 - s0 < kStep) {  // (the first and the last step of the range only)
      // of the lane's quad u, the nonzeros number [from, to) lie in [begin, s1)
      uint32_t inside = 0;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t p0 = s0 + static_cast<uint32_t>(u) * 4u * kWave + 4u * lane;
        const uint32_t from = begin > p0 ? (begin - p0 < 4u ? begin - p0 : 4u) : 0u;
        const uint32_t to = s1 > p0 ? (s1 - p0 < 4u ? s1 - p0 : 4u) : 0u;
        inside |= ((0xfu << from) & ~(0xfu << to) & 0xfu) << (4 * u);
      }
      hits &= inside;
      // the array's last, partial quad was not loaded: the lane whose quad it is probes its one to three columns
      const uint32_t tail = nnz & ~3u;
      if (tail != nnz && s1 == nnz && tail >= s0 && ((tail - s0) / 4u) % kWave == lane) {
        const uint32_t shift = (tail - s0) / (4u * kWave) * 4u;
        hits &= ~(0xfu << shift);
        for (uint32_t p = tail > begin ? tail : begin; p < nnz; ++p) {
          const uint32_t c = indices[p];
          hits |= __builtin_amdgcn_ubfe(s_bits[c >> 5], c, 1u) << (shift + (p - tail));
        }
      }
    }
    // where the lane's hits go in the step's sequence of hits
    const uint32_t mine = static_cast<uint32_t>(__popc(hits));
    const uint32_t incl = wave_inclusive_scan_u32(mine);
    const uint32_t total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), kWave - 1));
    // hits number base .. base + QUEUE - 1 of the step: the distance of each from s0 (256 u + 4 lane + t)
    auto fill_queue = [&](uint32_t base) {
      uint32_t m = hits, at = incl - mine;
      while (m != 0u) {
        const uint32_t b = static_cast<uint32_t>(__ffs(static_cast<int>(m))) - 1u;
        m &= m - 1u;
        if (at - base < QUEUE) s_queue[at - base] = static_cast<uint16_t>(((b >> 2) << 8) | (lane << 2) | (b & 3u));
        ++at;
      }
    };
    if (total != 0u && total <= QUEUE) fill_queue(0u);
    // windows of 64 rows from r on, until one reaches beyond the step (the first one was requested a step ago;
    // the loop reads it from LDS only, so that the wait for a further window's request stays on that path)
    store_window();
    for (;;) {
      __builtin_amdgcn_wave_barrier();
      const uint32_t lo = s_ptr[0], hi = s_ptr[kFlatEvRows];
      const uint32_t top = hi < s1 ? hi : s1;  // the window takes the hits at nonzeros [lo, top)
      for (uint32_t base = 0; base < total; base += QUEUE) {
        if (total > QUEUE) {
          __builtin_amdgcn_wave_barrier();
          fill_queue(base);
          __builtin_amdgcn_wave_barrier();
        }
        const uint32_t n = total - base < QUEUE ? total - base : QUEUE;
        for (uint32_t i = lane; i < n; i += kWave) {
          const uint32_t p = s0 + s_queue[i];
          if (p >= lo && p < top) {
            uint32_t k = 0;  // the last k < 64 with s_ptr[k] <= p
#pragma unroll
            for (uint32_t half = kFlatEvRows / 2; half != 0; half >>= 1)
              if (s_ptr[k + half] <= p) k += half;
            if constexpr (HETER) atomicAdd(&s_sum[k], static_cast<double>(data[p]));
            else atomicAdd(&s_sum[k], 1u);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
      // rows of the window that end inside the step (a prefix of the window) are stored
      const uint64_t row = static_cast<uint64_t>(r) + lane;
      const bool ended = row < r_end && s_ptr[lane + 1u] <= s1;
      const uint32_t n_ended = static_cast<uint32_t>(__popcll(__ballot(ended)));
      if (ended) {
        if constexpr (HETER) y[row] = static_cast<F>(s_sum[lane]);
        else y[row] = gathered_sum(w_homo, s_sum[lane]);
      }
      const A open = n_ended < kFlatEvRows ? s_sum[n_ended] : A(0);  // (wave uniform address: a broadcast)
      __builtin_amdgcn_wave_barrier();
      s_sum[lane] = A(0);
      r += n_ended;
      if (n_ended < kFlatEvRows || r >= r_end) {
        if (lane == 0) s_sum[0] = open;
        break;
      }
      load_window();
      store_window();
    }
    __builtin_amdgcn_wave_barrier();
    load_window();
    load_indices(s0 + static_cast<uint32_t>(DEPTH) * kStep, ci);
  };
  for (uint32_t s0 = first_step;;) {
    step(s0, ci0);
    if ((s0 += kStep) >= end) break;
    step(s0, ci1);
    if ((s0 += kStep) >= end) break;
    if constexpr (DEPTH == 3) {
      step(s0, ci2);
      if ((s0 += kStep) >= end) break;
    }
  }
}

// (Event input with the bitmap in LDS is meant to run two workgroups per CU: eight waves per SIMD, asked
// for here because the homogeneous-weight walks sit at exactly 64 registers and the hub-row pass behind
// them would otherwise raise the kernel's allocation to 66.)
// BITS: where the event probes go.  0: the event vector in global memory; 1: a bitmap in LDS;
// 2: a bitmap in LDS of more than 80 KB (one workgroup per CU; a kernel of its own, because its
// variants need more than the 64 registers that let two workgroups of the other cases share a CU).
template <typename F, typename VT, bool HETER, int MODE, int BITS>
__global__ __launch_bounds__(1024, (MODE == kEvent && BITS == 1) ? 8 : 4) void csr_gather_kernel(const F *__restrict__ data,
                                                          const uint32_t *__restrict__ indices,
                                                          const uint32_t *__restrict__ indptr,
                                                          const VT *__restrict__ x, F *__restrict__ y,
                                                          uint32_t n_row, uint32_t n_col, uint32_t skip_mean) {
  extern __shared__ __attribute__((aligned(16))) uint32_t s_bits[];
  uint32_t coarse_g = 0;
  if constexpr (MODE == kDense) {
    // BITS == 1: the dense vector itself is staged in LDS (the host checked that it fits), so the
    // per-nonzero gather is an LDS read instead of an L2 request and the kernel streams at HBM speed
    // BITS == 2: as much of it as fits; the kernel gathers the rest from L2 as without LDS
    if constexpr (BITS == 1 || BITS == 2) {
      VT *s_x = reinterpret_cast<VT *>(s_bits);
      const uint32_t fits = static_cast<uint32_t>(kLdsBitmapCap / sizeof(VT));
      coarse_g = n_col < fits ? n_col : fits;  // (the walks take it as the number of staged elements)
      for (uint32_t i = threadIdx.x; i < coarse_g; i += blockDim.x) s_x[i] = x[i];
      __syncthreads();
    }
  } else if constexpr (BITS == 3) {
    // x is the exact packed bitmap; the coarse one behind it goes to LDS
    coarse_g = coarse_shift(n_col);
    const uint32_t words = (coarse_bits(n_col, coarse_g) + 31u) >> 5;
    const uint32_t *coarse = reinterpret_cast<const uint32_t *>(x) + coarse_offset_words(n_col);
    for (uint32_t w = threadIdx.x; w < words; w += blockDim.x) s_bits[w] = coarse[w];
    __syncthreads();
  } else if constexpr (BITS != 0) {
    const uint32_t words = (n_col + 31u) >> 5;
    for (uint32_t w = threadIdx.x; w < words; w += blockDim.x) s_bits[w] = pack_events32<VT>(x, w << 5, n_col);
    __syncthreads();
  }
  if (n_row == 0) return;
  const uint32_t nnz = indptr[n_row];
  if (nnz == 0) {  // nothing to gather (and no valid element to point masked lanes at)
    for (uint32_t r = blockIdx.x * blockDim.x + threadIdx.x; r < n_row; r += gridDim.x * blockDim.x) y[r] = F(0);
    return;
  }
  // lanes per row from the mean row length
  const uint32_t mean = nnz / n_row;
  uint32_t gpb = 0, hub_len = 0;  // rows per workgroup and round of the walk chosen below, its longest row
  if constexpr (MODE == kDense && BITS == 0) {
    // (rows of `skip_mean` nonzeros or more on average: the launcher's other kernel has taken this matrix)
    if (skip_mean != 0 && mean >= skip_mean && nnz <= kFlatMaxNnz) return;
  }
  if constexpr (MODE == kDense && BITS == 2) {
    // (rows of 4 nonzeros or more but fewer than `skip_mean` on average: the flat walk has taken this matrix)
    if (skip_mean != 0 && mean >= 4u && mean < skip_mean && nnz <= kFlatMaxNnz) return;
  }
  if constexpr (MODE == kDense && BITS == 1) {
    // (nothing left to hide but the index and weight streams: the walks of the event gather)
    const VT *xs = reinterpret_cast<const VT *>(s_bits);
    if (mean >= 384) { gather_rows_wave<F, VT, HETER, MODE, BITS, 8>(data, indices, indptr, xs, y, n_row, s_bits, coarse_g); gpb = 1; hub_len = kHubSteps * 8 * kWave; }
    else if (mean >= 24) { gather_rows<F, VT, HETER, MODE, BITS, 8, 8>(data, indices, indptr, xs, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 8 * 8; }
    else if (mean >= 12) { gather_rows<F, VT, HETER, MODE, BITS, 4, 8>(data, indices, indptr, xs, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 8 * 4; }
    else { gather_rows<F, VT, HETER, MODE, BITS, 4, 4>(data, indices, indptr, xs, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 4 * 4; }
  } else if constexpr (MODE == kDense && BITS == 2) {
    if (mean >= 384) { gather_rows_wave<F, VT, HETER, MODE, BITS, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = 1; hub_len = kHubSteps * 8 * kWave; }
    else if (mean >= 24) { gather_rows<F, VT, HETER, MODE, BITS, 8, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 8 * 8; }
    else { gather_rows<F, VT, HETER, MODE, BITS, 4, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 8 * 4; }
  } else if constexpr (MODE == kEvent && (BITS == 2 || BITS == 3)) {
    // An event bitmap above 80 KB leaves room for one workgroup (16 waves) per CU only: every lane
    // then keeps 16 (rows under 48 nonzeros: 8) loads in flight instead of 2 to 8, in groups of
    // 8 or 4 lanes per row, or HBM sees too few requests (1e6 columns, 100 per row: 424 -> 164 us).
    if constexpr (BITS == 2) {
      // rows of 16 to 383 nonzeros on average: the flat walk over the nonzeros, which leaves no row to the pass below
      if (mean >= kFlatEvMinMean && mean < kFlatEvMaxMean && nnz <= kFlatMaxNnz && blockDim.x == kFlatEvWaves * kWave &&
          (reinterpret_cast<uintptr_t>(indices) & 15u) == 0) {
        gather_rows_flat_event<F, HETER, kFlatEvQuadsAlone, kFlatEvDepthAlone, kFlatEvQueueAlone>(
          data, indices, indptr, y, n_row, nnz, s_bits, s_bits + flat_event_lds_offset(n_col));
        return;
      }
    }
    if (mean >= 384) { gather_rows_wave<F, VT, HETER, MODE, BITS, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = 1; hub_len = kHubSteps * 8 * kWave; }
    else if (mean >= 48) { gather_rows<F, VT, HETER, MODE, BITS, 8, 16>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 16 * 8; }
    else { gather_rows<F, VT, HETER, MODE, BITS, 4, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 8 * 4; }
  } else {
    if constexpr (MODE == kEvent && BITS == 1 && HETER) {
      // The same walk within 64 registers, where the launcher left room for it behind the bitmap.  A wave's steps
      // form one chain of dependent round trips (row offsets, probes, search, the hits' weights), so the walk pays
      // from some 6,000 nonzeros per wave on: 500,000 x 500,000 with 100 per row 88 -> 76 us, 2,000,000 x 500,000
      // with 30 per row 116 -> 85 us, but 350,000 x 350,000 with 100 per row 56 -> 60 us.  With one weight the
      // row-wise walk has no weights to wait for and stays ahead (46 against 57 us for the first of these).
      if (mean >= kFlatEvMinMean && mean < kFlatEvSharedMaxMean && nnz >= kFlatEvSharedMinNnz && nnz <= kFlatMaxNnz &&
          blockDim.x == kFlatEvWaves * kWave && (reinterpret_cast<uintptr_t>(indices) & 15u) == 0 &&
          flat_event_shared_fits(n_row, n_col)) {
        gather_rows_flat_event<F, HETER, kFlatEvQuadsShared, kFlatEvDepthShared, kFlatEvQueueShared>(
          data, indices, indptr, y, n_row, nnz, s_bits, s_bits + flat_event_lds_offset(n_col));
        return;
      }
    }
    if (mean >= 384) { gather_rows_wave<F, VT, HETER, MODE, BITS, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = 1; hub_len = kHubSteps * 8 * kWave; }
    // (a dense vector is gathered from L2: for rows of 48 .. 191 nonzeros the pipelined 32-lane walk keeps more
    // of those gathers in flight than a wave per row does)
    else if (MODE == kEvent && mean >= 48u) { gather_rows<F, VT, HETER, MODE, BITS, 8, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 8 * 8; }
    else if (MODE == kDense && mean >= 192u) { gather_rows_wave<F, VT, HETER, MODE, BITS, 2>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = 1; hub_len = kHubSteps * 2 * kWave; }
    else if (mean >= 48) { gather_rows<F, VT, HETER, MODE, BITS, 32, 4>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 32; hub_len = kHubSteps * 4 * 32; }
    else if (MODE == kEvent && mean >= 24) { gather_rows<F, VT, HETER, MODE, BITS, 8, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 8 * 8; }
    else if (MODE == kEvent && mean >= 12) { gather_rows<F, VT, HETER, MODE, BITS, 4, 8>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 8 * 4; }
    else if (MODE == kEvent) { gather_rows<F, VT, HETER, MODE, BITS, 4, 4>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 4; hub_len = kHubSteps * 4 * 4; }
    else if (mean >= 24) { gather_rows<F, VT, HETER, MODE, BITS, 32, 2>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 32; hub_len = kHubSteps * 2 * 32; }
    else if (mean >= 12) { gather_rows<F, VT, HETER, MODE, BITS, 16, 2>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 16; hub_len = kHubSteps * 2 * 16; }
    else { gather_rows<F, VT, HETER, MODE, BITS, 8, 2>(data, indices, indptr, x, y, n_row, s_bits, coarse_g); gpb = blockDim.x / 8; hub_len = kHubSteps * 2 * 8; }
  }
  // the rows the walk left to the whole workgroup
  if constexpr (MODE == kDense && BITS == 1)
    gather_hub_rows<F, VT, HETER, MODE, BITS>(data, indices, indptr, reinterpret_cast<const VT *>(s_bits), y, n_row, s_bits,
                                              coarse_g, gpb, hub_len);
  else
    gather_hub_rows<F, VT, HETER, MODE, BITS>(data, indices, indptr, x, y, n_row, s_bits, coarse_g, gpb, hub_len);
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
// ------------------------------------------------------------------------------------------------
// scatter, small matrices with event input: one launch
// ------------------------------------------------------------------------------------------------
// Up to kSmallRows rows and kSmallCols columns (the synapses of one small population; the
// reference's own benchmark network has 4,000 x 4,000) a call is bound by how many dependent
// memory round trips and launches it needs, not by bandwidth.  One launch: workgroup b owns output
// window b (at most 16 windows).  Every workgroup loads ALL events and ALL row bounds at once (one
// round trip), lists the active rows in LDS, then groups of 16 lanes walk the listed rows (the
// indices of the next step, which may belong to the group's next row, are requested before this
// step's are used), add what falls into the window with LDS atomics (integer counts for a
// homogeneous weight) and the window is stored straight to y: no partial outputs to sum, no
// atomics on y, no zero fill.  Every workgroup streams all active nonzeros, so the time grows
// with the activity; the launcher takes this path for small matrices only.
constexpr uint32_t kSmallRows = 4096;
constexpr uint32_t kSmallCols = 8192;
constexpr uint32_t kSmallMaxWindows = 16;

template <typename F, typename VT, bool HETER>
__global__ __launch_bounds__(kWinThreads) void csr_scatter_small_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const VT *__restrict__ x, F *__restrict__ y, uint32_t n_row, uint32_t n_col, uint32_t win) {
  constexpr uint32_t kPer = kSmallRows / kWinThreads;  // rows tested per thread
  constexpr uint32_t G = 16, U = 8;                    // lanes per row, nonzeros per lane and step
  constexpr uint32_t kGroups = kWinThreads / G;
  __shared__ uint32_t s_start[kSmallRows], s_len[kSmallRows];
  __shared__ uint32_t s_count;
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  F *window = reinterpret_cast<F *>(smem_raw);
  uint32_t *cwindow = reinterpret_cast<uint32_t *>(smem_raw);
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  const uint32_t c0 = blockIdx.x * win;
  const uint32_t width = (c0 + win <= n_col) ? win : n_col - c0;

  // all events and row bounds: independent loads, issued together
  VT ev[kPer];
  uint32_t lo[kPer], hi[kPer];
#pragma unroll
  for (uint32_t k = 0; k < kPer; ++k) {
    const uint32_t r = k * kWinThreads + tid;
    ev[k] = VT(0);
    lo[k] = hi[k] = 0;
    if (r < n_row) {
      ev[k] = x[r];
      lo[k] = indptr[r];
      hi[k] = indptr[r + 1];
    }
  }
  const F w_homo = HETER ? F(0) : data[0];
  if (tid == 0) s_count = 0;
  for (uint32_t i = tid; i < width; i += kWinThreads) {
    if (HETER) window[i] = F(0);
    else cwindow[i] = 0u;
  }
  __syncthreads();
#pragma unroll
  for (uint32_t k = 0; k < kPer; ++k) {
    const bool on = is_event(ev[k]) && hi[k] > lo[k];
    const uint64_t mask = __ballot(on);
    uint32_t base = 0;
    if (lane == 0 && mask) base = atomicAdd(&s_count, static_cast<uint32_t>(__popcll(mask)));
    base = __builtin_amdgcn_readfirstlane(base);
    if (on) {
      const uint32_t at = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
      s_start[at] = lo[k];
      s_len[at] = hi[k] - lo[k];
    }
  }
  __syncthreads();
  const uint32_t count = s_count;

  // group `gid` walks listed rows gid, gid + kGroups, ... in steps of G * U nonzeros
  const uint32_t gid = tid / G, gl = tid % G;
  auto load_rel = [&](uint32_t start, uint32_t b0, uint32_t len, uint32_t (&rel)[U]) {
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t j = b0 + u * G + gl;
      rel[u] = 0xffffffffu;  // outside every window
      if (j < len) rel[u] = indices[start + j] - c0;
    }
  };
  uint32_t k = gid, start = 0, len = 0, b0 = 0;
  uint32_t rel[U];
  if (k < count) {
    start = s_start[k], len = s_len[k];
    load_rel(start, 0, len, rel);
  }
  while (k < count) {
    uint32_t nk = k, nstart = start, nlen = len, nb0 = b0 + G * U;
    if (nb0 >= len) {
      nk = k + kGroups, nb0 = 0;
      if (nk < count) nstart = s_start[nk], nlen = s_len[nk];
    }
    uint32_t nrel[U];
    if (nk < count) load_rel(nstart, nb0, nlen, nrel);
    if (HETER) {
      F w[U];
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        w[u] = F(0);
        if (rel[u] < width) w[u] = data[start + b0 + u * G + gl];
      }
#pragma unroll
      for (uint32_t u = 0; u < U; ++u)
        if (rel[u] < width) atomicAdd(&window[rel[u]], w[u]);
    } else {
#pragma unroll
      for (uint32_t u = 0; u < U; ++u)
        if (rel[u] < width) atomicAdd(&cwindow[rel[u]], 1u);
    }
    k = nk, start = nstart, len = nlen, b0 = nb0;
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) rel[u] = nrel[u];
  }
  __syncthreads();
  for (uint32_t i = tid; i < width; i += kWinThreads) {
    if (HETER) {
      y[c0 + i] = window[i];
    } else {
      y[c0 + i] = scattered_sum<F>(w_homo, cwindow[i]);  // the weight added once per synapse, as the reference adds it
    }
  }
}

template <typename F, typename VT, bool HETER, int MODE>
void launch_scatter(const ScratchSource &src, const F *data, const uint32_t *indices, const uint32_t *indptr,
                    const VT *x, F *y, uint32_t n_row, uint32_t n_col) {
  hipStream_t stream = src.stream;
  const char *target = MODE == kEvent ? "event scatter" : "transposed csr_matvec";
  if (n_col == 0) return;
  if (n_row == 0) {
    fill_zero(stream, y, n_col);
    return;
  }
  // Output windows in LDS (the path for narrow outputs, and the fallback of the event input when
  // the sorted scatter below has no scratch memory).  Every window's workgroup streams the column
  // indices of the active rows again, which is still far cheaper than one random global atomic per
  // nonzero (about 21 G/s) for a few windows; a wave walks its rows one after the other.
  using A = typename std::conditional<MODE == kDense, double, F>::type;  // window accumulators
  const size_t list_bytes = kWinMaxRows * (8 + (MODE == kDense ? sizeof(F) : 0));
  if constexpr (MODE == kEvent) {
    if (n_row <= kSmallRows && n_col <= kSmallCols) {
      uint32_t n_win = div_up(n_col, 256);
      if (n_win > kSmallMaxWindows) n_win = kSmallMaxWindows;
      const uint32_t win = div_up(n_col, n_win);
      n_win = div_up(n_col, win);
      hipLaunchKernelGGL((csr_scatter_small_kernel<F, VT, HETER>), dim3(n_win), dim3(kWinThreads),
                         static_cast<size_t>(win) * sizeof(F), stream, data, indices, indptr, x, y, n_row, n_col, win);
      return;
    }
  }
  const uint32_t win_cap = static_cast<uint32_t>((static_cast<size_t>(128) * 1024) / sizeof(A));
  const uint32_t n_win = div_up(n_col, win_cap);
  NnzGate direct_gate = kAlways;
  auto round_up = [](size_t v) { return (v + 255) / 256 * 256; };
  // Event input, 4,097 to 32,768 rows and an output of at most two windows of 7,424 columns: the flat walk over
  // the active rows' nonzeros into LDS windows (csr_bin_scatter.hip), whose workgroups find the active rows
  // themselves.  Two launches, where the sorted scatter below needs three and the window kernel further down,
  // which needs two as well, has 16 workgroups walk their rows one after the other (32,000 x 8,192 with 1,000
  // per row at 20 % events: 545 us against 31).  (Not from a fixed arena: the walks below need less scratch
  // memory there.)
  if constexpr (MODE == kEvent && (sizeof(VT) == 1 || std::is_floating_point<VT>::value)) {
    if (!src.fixed() && n_row > kSmallRows && window_event_scatter_self_usable(n_row, n_col, HETER)) {
      const size_t need = window_event_scatter_bytes<F>(n_col);
      size_t got = 0;
      unsigned char *ws = static_cast<unsigned char *>(src.request(need, need, &got));
      uint32_t *counters = ws ? src.counters() : nullptr;
      if (ws != nullptr && counters != nullptr) {
        if (window_event_scatter<F>(stream, data, HETER, indices, indptr, y, n_row, n_col, counters, nullptr, 0u, ws, got,
                                    static_cast<const void *>(x), static_cast<uint32_t>(sizeof(VT))))
          return;
      } else {
        if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // during a capture: the error stands
        bpl_clear_error();  // no scratch memory: the paths below need less or none
      }
    }
  }
  // Event input and more than 8,192 outputs: the active rows' nonzeros are flattened and sorted
  // coarsely by output window instead (csr_bin_scatter.hip), at a cost that neither grows with the
  // number of windows nor with the number of rows a wave would have to walk in turn.
  const bool listed_windows = MODE == kEvent && !src.fixed() && n_row > kSmallRows && window_event_scatter_usable<F>(n_row, n_col, HETER);
  if (MODE == kEvent && n_col > 8192 && bin_event_scatter_usable<F>(n_col) && !listed_windows) {
    const size_t list_sz = round_up(static_cast<size_t>(n_row) * sizeof(uint2));
    size_t got = 0;
    unsigned char *ws = static_cast<unsigned char *>(src.request(list_sz + bin_event_scatter_bytes<F>(n_row, n_col),
                                                                 list_sz + bin_event_scatter_min_bytes<F>(n_col), &got));
    uint32_t *counters = ws ? src.counters() : nullptr;
    if (ws != nullptr && counters != nullptr) {
      uint2 *active_list = reinterpret_cast<uint2 *>(ws);
      // (a fixed arena is shared by every call on the device and keeps the last call's contents)
      if (src.fixed()) fill_zero(stream, counters, 2u);
      // the kernel that lists the active rows also zeroes the windows' fill counters and, unless
      // the output is much longer than the input, y
      const unsigned collectors = collect_workgroups<F, VT, MODE>(n_row);
      const bool fold_zero = n_col <= 32ull * collectors * kWinThreads;
      if (!fold_zero) fill_zero(stream, y, n_col);
      launch_collect<F, VT, MODE>(stream, indptr, x, n_row, counters, active_list, static_cast<F *>(nullptr), kAlways,
                                  reinterpret_cast<uint32_t *>(ws + list_sz),
                                  static_cast<uint32_t>(kBinEventFillBytes / sizeof(uint32_t)), y,
                                  fold_zero ? n_col : 0u);
      if (bin_event_scatter<F>(stream, data, HETER, indices, indptr, y, n_row, n_col, counters, active_list, n_row,
                               ws + list_sz, got - list_sz))
        return;
      fill_zero(stream, counters, 1u);  // (the sort could not run: the list is not used)
    } else {
      if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // beyond a fixed arena, or during a capture: the error stands
      bpl_clear_error();  // no scratch memory: the paths below need less or none
    }
  }
  // Event input, more rows and an output of one window: the same walk over a device list of the active rows.
  if (listed_windows) {
    const size_t list_sz = round_up(static_cast<size_t>(n_row) * sizeof(uint2));
    const size_t need = list_sz + window_event_scatter_bytes<F>(n_col);
    size_t got = 0;
    unsigned char *ws = static_cast<unsigned char *>(src.request(need, need, &got));
    uint32_t *counters = ws ? src.counters() : nullptr;
    if (ws != nullptr && counters != nullptr) {
      uint2 *active_list = reinterpret_cast<uint2 *>(ws);
      launch_collect<F, VT, MODE>(stream, indptr, x, n_row, counters, active_list, static_cast<F *>(nullptr), kAlways,
                                  static_cast<uint32_t *>(nullptr), 0u, static_cast<F *>(nullptr), 0u);
      if (window_event_scatter<F>(stream, data, HETER, indices, indptr, y, n_row, n_col, counters, active_list, n_row,
                                  ws + list_sz, got - list_sz))
        return;
      fill_zero(stream, counters, 1u);  // (the walk could not run: the list is not used)
    } else {
      if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // during a capture: the error stands
      bpl_clear_error();  // no scratch memory: the paths below need less or none
    }
  }
  if (n_win <= (MODE == kEvent ? 32u : 4u)) {
    const uint32_t win = div_up(n_col, n_win);
    // about one workgroup per CU in total, at least 64 rows each
    unsigned want_groups = static_cast<unsigned>(device_info().num_cu) / n_win;
    if (want_groups == 0) want_groups = 1;
    // small outputs: at most 16 row groups (their slices are summed by the second kernel)
    // (dense input: every row is active and a wave walks its rows one after the other, so more groups)
    const unsigned small_groups = MODE == kEvent ? 16 : 64;
    if (static_cast<size_t>(n_col) * 16 <= 131072 && n_row <= 16 * kWinMaxRows && want_groups > small_groups)
      want_groups = small_groups;
    uint32_t rows_per_wg = div_up(n_row, want_groups);
    if (rows_per_wg < 64) rows_per_wg = 64;
    // Large matrices: the active rows are first gathered into one list (a launch of its own) and
    // the row groups share the list evenly; small ones find their active rows themselves.
    const bool use_list = n_row > 16 * kWinMaxRows;
    const unsigned groups = use_list ? want_groups : div_up(n_row, rows_per_wg);
    // The window kernel hands whole rows to waves, one after the other: with more than a few
    // windows it only beats the direct atomics when rows are long (64 nonzeros on average).
    NnzGate window_gate = kAlways;
    bool usable = true;
    if (n_win > 4) {
      const unsigned long long min_nnz = 64ull * n_row;
      if (min_nnz > 0xffffffffull) {
        usable = false;
      } else {
        window_gate = {static_cast<uint32_t>(min_nnz), 0xffffffffu};
        direct_gate = {0u, static_cast<uint32_t>(min_nnz) - 1u};
      }
    }
    const size_t lds = static_cast<size_t>(win) * sizeof(A) + list_bytes;
    auto kernel = csr_scatter_window_kernel<F, VT, HETER, MODE, A>;
    static thread_local size_t attr_set_for = 0;
    if (usable && lds > 64 * 1024 && attr_set_for < lds) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds)) == hipSuccess)
        attr_set_for = lds;
      else
        (void)hipGetLastError();
    }
    if (usable && (lds <= 64 * 1024 || attr_set_for >= lds)) {
      // Per-row-group partial outputs in scratch memory, summed by a second kernel (no global
      // atomics, no zero fill), as long as they stay small; else atomics into the zeroed y.
      const size_t partial_bytes = static_cast<size_t>(groups) * n_col * sizeof(F);
      bool want_partial = groups > 1 && partial_bytes <= (static_cast<size_t>(64) << 20);
      // workspace: [active-row list][dense mode: their input values][partial outputs]
      const size_t list_off = 0, list_sz = use_list ? round_up(static_cast<size_t>(n_row) * sizeof(uint2)) : 0;
      const size_t scale_sz = (use_list && MODE == kDense) ? round_up(static_cast<size_t>(n_row) * sizeof(F)) : 0;
      const size_t partial_off = list_sz + scale_sz;
      const size_t ws_bytes = partial_off + (want_partial ? partial_bytes : 0);
      size_t got = 0;
      unsigned char *ws = ws_bytes ? static_cast<unsigned char *>(src.request(ws_bytes, partial_off, &got)) : nullptr;
      if (ws != nullptr && got < ws_bytes) want_partial = false;  // (a fixed arena too small for the partial outputs)
      uint32_t *counters = (use_list && (ws != nullptr || ws_bytes == 0)) ? src.counters() : nullptr;
      if (ws_bytes != 0 && (ws == nullptr || (use_list && counters == nullptr))) {
        if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // beyond a fixed arena, or during a capture: the error stands
        // no scratch memory: the direct kernel needs none
        bpl_clear_error();
        fill_zero(stream, y, n_col);
        hipLaunchKernelGGL((csr_scatter_kernel<F, VT, HETER, MODE>), dim3(div_up(n_row, kScatterRows)),
                           dim3(kScatterThreads), 0, stream, data, indices, indptr, x, y, n_row, kAlways);
        return;
      }
      F *partial = want_partial ? reinterpret_cast<F *>(ws + partial_off) : nullptr;
      uint2 *active_list = use_list ? reinterpret_cast<uint2 *>(ws + list_off) : nullptr;
      F *active_scales = scale_sz ? reinterpret_cast<F *>(ws + list_sz) : nullptr;
      uint32_t *active_count = use_list ? counters : nullptr;
      const bool gated = n_win > 4;
      if (use_list && src.fixed()) fill_zero(stream, counters, 2u);
      if (partial == nullptr || gated) fill_zero(stream, y, n_col);
      if (use_list)
        launch_collect<F, VT, MODE>(stream, indptr, x, n_row, active_count, active_list, active_scales, window_gate,
                                    static_cast<uint32_t *>(nullptr), 0u, static_cast<F *>(nullptr), 0u);
      hipLaunchKernelGGL(kernel, dim3(groups * n_win), dim3(kWinThreads), lds, stream, data, indices, indptr, x, y,
                         n_row, n_col, rows_per_wg, win, n_win, partial, window_gate, active_count,
                         active_list, active_scales);
      // the list's counter goes back to zero: by the summing kernel, else by a fill of its own
      constexpr bool kCount = !HETER && MODE == kEvent;  // the windows count synapses of the homogeneous weight
      if (partial != nullptr) {
        hipLaunchKernelGGL((sum_partials_kernel<F, kCount>), dim3(div_up(n_col, 256)), dim3(256), 0, stream,
                           static_cast<const F *>(partial), y, n_col, groups, indptr, n_row, window_gate, active_count,
                           data);
      } else {
        if (use_list) fill_zero(stream, active_count, 1u);
        if (kCount)  // y holds the counts the windows added
          hipLaunchKernelGGL(counts_to_sums_kernel<F>, dim3(div_up(n_col, 256)), dim3(256), 0, stream, y, n_col, data,
                             indptr, n_row, window_gate);
      }
      if (!gated) return;
    } else {
      direct_gate = kAlways;
      fill_zero(stream, y, n_col);
    }
  } else {
    fill_zero(stream, y, n_col);
  }
  hipLaunchKernelGGL((csr_scatter_kernel<F, VT, HETER, MODE>), dim3(div_up(n_row, kScatterRows)),
                     dim3(kScatterThreads), 0, stream, data, indices, indptr, x, y, n_row, direct_gate);
}

template <typename F, typename VT, bool HETER, int MODE, int BITS>
bool launch_gather_impl(const char *target, hipStream_t stream, const F *data, const uint32_t *indices,
                        const uint32_t *indptr, const VT *x, F *y, uint32_t n_row, uint32_t n_col,
                        size_t lds_bytes, uint32_t skip_mean = 0) {
  auto kernel = csr_gather_kernel<F, VT, HETER, MODE, BITS>;
  // Small problems: 256-thread workgroups, one wave per row at most.  Large ones: 1024-thread
  // persistent workgroups so that few copies of the event bitmap are built.
  // (Few rows over many columns, or an LDS image of more than 16 KB per workgroup: the large ones too.)
  const bool wide = n_col > kHubSteps * 8 * kWave;  // rows can be long enough to go to whole workgroups
  const int block = (n_row >= 16384 || lds_bytes > 16 * 1024 || (wide && n_row < 2048)) ? 1024 : 256;
  // The occupancy query is the same for every call with the same LDS size: remember the last one.
  struct Cached {
    size_t lds_bytes;
    int block;
    int per_cu;
  };
  static thread_local Cached cached = {~size_t(0), 0, 0};
  if (cached.lds_bytes != lds_bytes || cached.block != block) {
    if (lds_bytes > 64 * 1024) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds_bytes)) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
    }
    int q = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, reinterpret_cast<const void *>(kernel), block,
                                                     lds_bytes) != hipSuccess || q < 1) {
      (void)hipGetLastError();
      q = 1;
    }
    cached = {lds_bytes, block, q};
  }
  const int per_cu = cached.per_cu;
  const unsigned resident = static_cast<unsigned>(device_info().num_cu) * static_cast<unsigned>(per_cu);
  unsigned needed = div_up(n_row, block / kWave);  // one wave per row
  // Few rows over many columns may all be long enough to go to whole workgroups, one row each (gather_hub_rows;
  // the row lengths are known on the device only): then a workgroup per row, or most of the device has no row.
  if (wide && n_row < 2048) needed = n_row;
  const unsigned grid = needed < resident ? (needed ? needed : 1u) : resident;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), lds_bytes, stream, data, indices, indptr, x, y, n_row,
                     n_col, skip_mean);
  return check_launch(target);
}

template <typename F, typename VT, bool HETER, int MODE>
void launch_gather(const char *target, const ScratchSource &src, const F *data, const uint32_t *indices,
                   const uint32_t *indptr, const VT *x, F *y, uint32_t n_row, uint32_t n_col) {
  hipStream_t stream = src.stream;
  if (n_row == 0) return;
  if constexpr (MODE == kEvent && !std::is_same<VT, PackedBits>::value) {
    // A bitmap that does not fit LDS (more than 1.3 million columns): two levels, the exact one in
    // global memory and a coarse one (one bit per 2^g columns) for LDS, both built here.
    if ((static_cast<size_t>(n_col) + 31) / 32 * 4 > kLdsEventBitmapCap) {
      const uint32_t g = coarse_shift(n_col);
      const uint32_t n_words = (n_col + 31u) / 32u, off = coarse_offset_words(n_col);
      const uint32_t c_words = (coarse_bits(n_col, g) + 31u) / 32u;
      uint32_t *bits = static_cast<uint32_t *>(src.request((static_cast<size_t>(off) + c_words + 1) * sizeof(uint32_t)));
      if (bits != nullptr) {
        pack_event_bitmap<VT>(stream, x, n_col, bits);
        hipLaunchKernelGGL(coarsen_bitmap_kernel, dim3(div_up(c_words, 256)), dim3(256), 0, stream, bits, n_words, g,
                           bits + off, c_words);
        if (launch_gather_impl<F, PackedBits, HETER, MODE, 3>(target, stream, data, indices, indptr,
                                                              reinterpret_cast<const PackedBits *>(bits), y, n_row,
                                                              n_col, static_cast<size_t>(c_words) * 4))
          return;
      }
      if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // beyond a fixed arena, or during a capture: the error stands
      bpl_clear_error();
    }
  }
  if constexpr (MODE == kEvent && !std::is_same<VT, PackedBits>::value) {
    // Wide event types: every persistent workgroup would read the whole vector (4 or 8 bytes per
    // element) to build its bitmap; pack it once instead and hand the words to the kernels.  Byte events
    // likewise from 655,360 columns on (a bitmap of more than 80 KB, one workgroup per CU: 256 workgroups that
    // each read a megabyte of events take longer than one small kernel and 125 KB per workgroup).
    const size_t words = (static_cast<size_t>(n_col) + 31) / 32;
    uint32_t *bits = (sizeof(VT) > 1 || words * 4 > kLdsSharedBitmapCap)
                         ? static_cast<uint32_t *>(src.request((words + 1) * sizeof(uint32_t)))
                         : nullptr;
    if (sizeof(VT) == 1 && words * 4 <= kLdsSharedBitmapCap) {
      // (byte events and a bitmap that leaves room for two workgroups per CU: they pack it themselves)
    } else if (bits != nullptr) {
      pack_event_bitmap<VT>(stream, x, n_col, bits);
      launch_gather<F, PackedBits, HETER, MODE>(target, src, data, indices, indptr,
                                                reinterpret_cast<const PackedBits *>(bits), y, n_row, n_col);
      return;
    } else {
      if (src.failure_is_final()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // beyond a fixed arena, or during a capture: the error stands
      bpl_clear_error();
    }
  }
  if (MODE == kEvent) {
    const size_t lds_bytes = (static_cast<size_t>(n_col) + 31) / 32 * 4;
    const size_t lds_cap = kLdsEventBitmapCap;
    if (lds_bytes <= lds_cap) {
      // (behind the bitmap: the memory of the flat walk over short rows, where it fits and is used)
      const size_t walk_at = static_cast<size_t>(flat_event_lds_offset(n_col)) * 4;
      const size_t shared_bytes =
        HETER && flat_event_shared_fits(n_row, n_col) ? walk_at + flat_event_lds_bytes(kFlatEvQueueShared) : lds_bytes;
      const bool ok = lds_bytes > kLdsSharedBitmapCap  // (two workgroups per CU below)
                          ? launch_gather_impl<F, VT, HETER, MODE, 2>(target, stream, data, indices, indptr, x, y, n_row,
                                                                      n_col, walk_at + flat_event_lds_bytes(kFlatEvQueueAlone))
                          : launch_gather_impl<F, VT, HETER, MODE, 1>(target, stream, data, indices, indptr, x, y, n_row,
                                                                      n_col, shared_bytes);
      if (ok) return;
      bpl_clear_error();
    }
  }
  if constexpr (MODE == kDense) {
    // A dense vector that fits LDS beside nothing else (up to 40,704 floats), under persistent
    // workgroups (few copies): staged there.  Gathers from L2 cap the product at about 140 G nonzeros
    // per second whatever the vector's size; from LDS the index and weight streams are the limit.
    // (From 2,048 rows: 10,000 x 10,000 with 1,000 per row 28 -> 19 us, 8,000 x 30,000 with 300 per row 15 -> 12 us;
    // a matrix of few nonzeros pays up to a microsecond for the copies, 12,000 x 38,000 with 50 per row 8.8 -> 9.3 us.)
    const size_t lds_bytes = static_cast<size_t>(n_col) * sizeof(VT);
    if (n_row >= 2048 && n_col > 0 && lds_bytes <= kLdsBitmapCap) {
      if (launch_gather_impl<F, VT, HETER, MODE, 1>(target, stream, data, indices, indptr, x, y, n_row, n_col,
                                                    lds_bytes))
        return;
      bpl_clear_error();
    } else if (n_row >= 16384 && lds_bytes <= 4 * kLdsBitmapCap) {
      // up to four times that: the part that fits is staged (one workgroup per CU), which takes a
      // quarter or more of the gathers off the L2.  Its walk is row-wise: rows of 4 to 23 nonzeros on average
      // go to the flat walk over the nonzeros instead (the mean is known on the device only: both are enqueued).
      constexpr uint32_t kStagedMinMean = 24;
      bool flat_takes_short_rows = false;
      if constexpr (std::is_same<F, VT>::value) {
        const FlatGather flat = csr_flat_gather<F>(target, stream, data, HETER, indices, indptr, x, y, n_row, 4u, kStagedMinMean);
        if (flat == FlatGather::kFailed) {
          if (scratch_refused_by_capture()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // (the error stands: a graph must not record a slower path)
          bpl_clear_error();
        }
        flat_takes_short_rows = flat == FlatGather::kEnqueued;
      }
      if (launch_gather_impl<F, VT, HETER, MODE, 2>(target, stream, data, indices, indptr, x, y, n_row, n_col,
                                                    kLdsBitmapCap, flat_takes_short_rows ? kStagedMinMean : 0u))
        return;
      bpl_clear_error();
    }
    if constexpr (std::is_same<F, VT>::value) {
      // A longer vector is gathered from L2.  Rows of 4 nonzeros or more on average: the flat walk over the
      // nonzeros with 16-byte loads of the index and weight streams (csr_flat_gather.hip; 4,000,000 rows of 8:
      // 224 against 304 us, 2,000,000 rows of 20: 255 against 348 us); shorter ones: the walks below.  The
      // mean is known on the device only, so both are enqueued and one returns at once.  (Under 16,384 rows
      // the walks below stay: with 2,000 rows of 40,000 and a vector of 12 MB the walk that keeps a row's
      // gathers together takes 507 us, the flat one 835; only matrices of a few hundred rows that are
      // nearly dense would gain, and small ones would pay for a launch that returns at once.)
      constexpr uint32_t kFlatMinMean = 4;
      if (n_row >= 16384 && n_col > 0) {
        const FlatGather flat =
          csr_flat_gather<F>(target, stream, data, HETER, indices, indptr, x, y, n_row, kFlatMinMean, 0xffffffffu);
        if (flat == FlatGather::kEnqueued) {
          launch_gather_impl<F, VT, HETER, MODE, 0>(target, stream, data, indices, indptr, x, y, n_row, n_col, 0,
                                                    kFlatMinMean);
          return;
        }
        if (flat == FlatGather::kFailed) {
          if (scratch_refused_by_capture()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // (the error stands: a graph must not record a slower path)
          bpl_clear_error();
        }
      }
    }
  }
  launch_gather_impl<F, VT, HETER, MODE, 0>(target, stream, data, indices, indptr, x, y, n_row, n_col, 0);
}

// event_csr_matvec: buffers = [data, indices, indptr, events, out]
template <typename F, typename VT, bool HETER>
void event_csr_matvec_entry(const char *target, const ScratchSource &src, void **buffers, const char *opaque,
                            size_t opaque_len) {
  bpl_twouint_onebool_descriptor d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  const F *data = static_cast<const F *>(buffers[0]);
  const uint32_t *indices = static_cast<const uint32_t *>(buffers[1]);
  const uint32_t *indptr = static_cast<const uint32_t *>(buffers[2]);
  const VT *events = static_cast<const VT *>(buffers[3]);
  F *out = static_cast<F *>(buffers[4]);
  if (d.transpose) {
    launch_scatter<F, VT, HETER, kEvent>(src, data, indices, indptr, events, out, d.n_row, d.n_col);
    check_launch(target);
  } else {
    launch_gather<F, VT, HETER, kEvent>(target, src, data, indices, indptr, events, out, d.n_row, d.n_col);
  }
}

// csr_matvec: buffers = [data, indices, indptr, (row_blocks,) vector, out]
template <typename F, bool HETER, bool TRANSPOSE>
void csr_matvec_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque,
                      size_t opaque_len, int vector_slot) {
  bpl_double_size_descriptor d;
  uint32_t nnz = 0;  // known only to the transposed targets' longer descriptor
  begin_call();
  if (TRANSPOSE && opaque != nullptr && opaque_len == sizeof(bpl_csr_transpose_descriptor)) {
    bpl_csr_transpose_descriptor t;
    std::memcpy(&t, opaque, sizeof(t));
    d.n_row = t.n_row, d.n_col = t.n_col, nnz = t.nnz;
  } else if (!unpack(target, opaque, opaque_len, &d)) {
    return;
  }
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  const F *data = static_cast<const F *>(buffers[0]);
  const uint32_t *indices = static_cast<const uint32_t *>(buffers[1]);
  const uint32_t *indptr = static_cast<const uint32_t *>(buffers[2]);
  const F *vec = static_cast<const F *>(buffers[vector_slot]);
  F *out = static_cast<F *>(buffers[vector_slot + 1]);
  if (TRANSPOSE) {
    // Outputs beyond one float64 LDS window: sort the products coarsely.  (With every row active each
    // further window means another pass over the whole matrix; the windows remain for matrices too
    // small to sort or of unknown size, direct atomics beyond four windows.)
    const uint32_t plain_windows = div_up(d.n_col, static_cast<uint32_t>((128u * 1024u) / sizeof(double)));
    if (plain_windows > kFlatWindowMaxSlices && d.n_row > 0 && bin_scatter_usable<F>(d.n_col, nnz)) {
      if (bin_scatter<F>(target, stream, data, HETER, indices, indptr, vec, out, d.n_row, d.n_col, nnz)) return;
      if (scratch_refused_by_capture()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // (the error stands)
    }
    // One or two windows and a matrix worth a chip full of workgroups: the flat walk over the nonzeros, once per
    // window (167 and 330 us at 1e8 nonzeros; the sort takes 420).  (Smaller ones, and callers whose descriptor
    // does not say how many nonzeros there are, keep the walk that hands rows to waves.)
    if (plain_windows <= kFlatWindowMaxSlices && nnz >= (1u << 20)) {
      if (flat_window_scatter<F>(target, stream, data, HETER, indices, indptr, vec, out, d.n_row, d.n_col)) return;
      if (scratch_refused_by_capture()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");  // (the error stands)
    }
    launch_scatter<F, F, HETER, kDense>(ScratchSource{stream}, data, indices, indptr, vec, out, d.n_row, d.n_col);
    check_launch(target);
  } else {
    launch_gather<F, F, HETER, kDense>(target, ScratchSource{stream}, data, indices, indptr, vec, out, d.n_row, d.n_col);
  }
}


// ------------------------------------------------------------------------------------------------
// Batched event gather: one matrix, several event vectors
// (brainpylib/_src/event_ops/event_csr_matvec.py:152-193 is the CPU kernel of the batching
// primitive; the reference has no GPU kernel for it, :227-229).
// The column indices are streamed once per tile of kBatchTile event vectors: a byte per column
// holds the tile's event flags, so one probe answers for eight vectors.
// ------------------------------------------------------------------------------------------------
constexpr int kBatchTile = 8;

// mask[t * stride + c] bit b = events[((8 t + b) % events_batch) * n_col + c] != 0, for 8 t + b < batch
template <typename VT>
__global__ __launch_bounds__(256) void pack_event_masks_kernel(const VT *__restrict__ events,
                                                               uint8_t *__restrict__ mask, uint32_t n_col,
                                                               uint32_t stride, uint32_t batch,
                                                               uint32_t events_batch) {
  const uint32_t c = blockIdx.x * 256u + threadIdx.x;
  const uint32_t t = blockIdx.y;
  if (c >= n_col) return;
  uint32_t m = 0;
#pragma unroll
  for (uint32_t b = 0; b < kBatchTile; ++b) {
    const uint32_t bi = t * kBatchTile + b;
    if (bi < batch && is_event(events[static_cast<size_t>(bi % events_batch) * n_col + c])) m |= 1u << b;
  }
  mask[static_cast<size_t>(t) * stride + c] = static_cast<uint8_t>(m);
}

// Sums eight values per lane over aligned groups of G lanes (G = 8, 16, 32 or 64), halving the
// number of live values at each of the first three exchange steps.  Lane gl of the group ends
// up with the group total of value number k = (bit G/2 of gl)*4 + (bit G/4)*2 + (bit G/8);
// the lanes whose low bits (below G/8) are zero are the ones meant to use it.
template <int G, typename T>
__device__ __forceinline__ T group_sum8(const T (&v)[8], uint32_t gl, uint32_t *k) {
  constexpr int o1 = G / 2, o2 = G / 4, o3 = G / 8;
  const bool h1 = gl & o1, h2 = gl & o2, h3 = gl & o3;
  T a[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const T send = h1 ? v[i] : v[i + 4];
    const T keep = h1 ? v[i + 4] : v[i];
    a[i] = keep + __shfl_xor(send, o1, kWave);
  }
  T b[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const T send = h2 ? a[i] : a[i + 2];
    const T keep = h2 ? a[i + 2] : a[i];
    b[i] = keep + __shfl_xor(send, o2, kWave);
  }
  T c;
  {
    const T send = h3 ? b[0] : b[1];
    const T keep = h3 ? b[1] : b[0];
    c = keep + __shfl_xor(send, o3, kWave);
  }
#pragma unroll
  for (int off = o3 / 2; off > 0; off >>= 1) c += __shfl_xor(c, off, kWave);
  *k = (h1 ? 4u : 0u) | (h2 ? 2u : 0u) | (h3 ? 1u : 0u);
  return c;
}

// Tables in LDS that turn four bits of a column's mask into what the lanes add, instead of eight masked
// additions per nonzero (32 of the walk's ~40 instructions):
//   ones[h][n][k]   1.0 where bit k of nibble n is set, else 0.0 (h = 0: bits 0..3, h = 1: bits 4..7): a weight
//                   is added to the eight accumulators with eight fused multiply-adds by 1.0 or 0.0, which is the
//                   masked addition bit for bit (v * 1.0 = v, v * 0.0 = +-0) as long as v is finite;
//   spread[n]       bit k of nibble n in byte k: a homogeneous weight's eight synapse counts advance with two
//                   32-bit additions (four byte counters each), emptied into the full counters every 255 steps.
// A row is 48 bytes so that the rows of the empty nibble and of the one-bit nibbles lie in different banks.
struct BatchTables {
  double ones[2][16][6];
  uint32_t spread[16];
};
__device__ __forceinline__ void fill_batch_tables(BatchTables *t) {
  if (threadIdx.x < 128u) {
    const uint32_t h = threadIdx.x >> 6, n = (threadIdx.x >> 2) & 15u, k = threadIdx.x & 3u;
    t->ones[h][n][k] = ((n >> k) & 1u) ? 1.0 : 0.0;
  }
  if (threadIdx.x < 16u) {
    const uint32_t n = threadIdx.x;
    t->spread[n] = (n & 1u) | ((n & 2u) << 7) | ((n & 4u) << 14) | ((n & 8u) << 21);
  }
}

template <typename F, bool HETER, bool LDS_MASK, int G, int U>
__device__ __forceinline__ void gather_rows_batched(const F *__restrict__ data,
                                                    const uint32_t *__restrict__ indices,
                                                    const uint32_t *__restrict__ indptr,
                                                    const uint8_t *__restrict__ mask, F *__restrict__ y,
                                                    uint32_t n_row, uint32_t batch, uint32_t tile,
                                                    const BatchTables *__restrict__ tab) {
  const uint32_t gl = threadIdx.x & (G - 1);
  const uint32_t groups_per_block = blockDim.x / G;
  const uint32_t total_groups = gridDim.x * groups_per_block;
  const F w_homo = HETER ? F(0) : data[0];
  for (uint32_t row = blockIdx.x * groups_per_block + threadIdx.x / G; row < n_row; row += total_groups) {
    uint32_t start = indptr[row], end = indptr[row + 1];
    if (G == kWave) {
      start = __builtin_amdgcn_readfirstlane(start);
      end = __builtin_amdgcn_readfirstlane(end);
    }
    double acc[kBatchTile];
    uint32_t cnt[kBatchTile];
#pragma unroll
    for (int k = 0; k < kBatchTile; ++k) acc[k] = 0.0, cnt[k] = 0u;
    uint32_t bytes_lo = 0, bytes_hi = 0, since = 0;  // homogeneous weight: four byte counters each
    auto empty_bytes = [&]() {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        cnt[k] += (bytes_lo >> (8 * k)) & 0xffu;
        cnt[k + 4] += (bytes_hi >> (8 * k)) & 0xffu;
      }
      bytes_lo = bytes_hi = since = 0;
    };
    // software pipeline: the column indices of the next step are requested before this step's
    // probes and weights are waited for
    uint32_t col[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = start + u * G + gl;
      col[u] = j < end ? (G == kWave ? stream_load(indices + j) : indices[j]) : 0u;
    }
    for (uint32_t base = start; base < end; base += U * G) {
      uint32_t coln[U];
      const uint32_t nbase = base + U * G;
      if (nbase < end) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t j = nbase + u * G + gl;
          coln[u] = j < end ? (G == kWave ? stream_load(indices + j) : indices[j]) : 0u;
        }
      }
      uint32_t m[U];
      F val[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t j = base + u * G + gl;
        m[u] = j < end ? static_cast<uint32_t>(mask[col[u]]) : 0u;
      }
      if (HETER) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t j = base + u * G + gl;
          val[u] = F(0);
          if (m[u] != 0u) val[u] = G == kWave ? stream_load(data + j) : data[j];
        }
      }
      if constexpr (HETER) {
        // (0 * inf and 0 * NaN are not 0: a step that holds a weight that is not finite takes the masked additions)
        bool finite = true;
#pragma unroll
        for (int u = 0; u < U; ++u) finite = finite && (val[u] - val[u] == F(0));
        if (__builtin_amdgcn_ballot_w64(!finite) == 0ull) {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const double v = static_cast<double>(val[u]);
            const double *lo = tab->ones[0][m[u] & 15u], *hi = tab->ones[1][m[u] >> 4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              acc[k] = __fma_rn(v, lo[k], acc[k]);
              acc[k + 4] = __fma_rn(v, hi[k], acc[k + 4]);
            }
          }
        } else {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            // v or +0.0 by bit k of the mask: sign-extend the bit into a word mask, AND both halves
            const double v = static_cast<double>(val[u]);
            const int lo = __double2loint(v), hi = __double2hiint(v);
#pragma unroll
            for (int k = 0; k < kBatchTile; ++k) {
              const int t = __builtin_amdgcn_sbfe(static_cast<int>(m[u]), k, 1);
              acc[k] += __hiloint2double(hi & t, lo & t);
            }
          }
        }
      } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          bytes_lo += tab->spread[m[u] & 15u];
          bytes_hi += tab->spread[m[u] >> 4];
        }
        since += U;
        if (since > 255u - U) empty_bytes();
      }
      if (nbase < end) {
#pragma unroll
        for (int u = 0; u < U; ++u) col[u] = coln[u];
      }
    }
    uint32_t k;
    F result;
    if (HETER) {
      result = static_cast<F>(group_sum8<G>(acc, gl, &k));
    } else {
      empty_bytes();
      const uint32_t n = group_sum8<G>(cnt, gl, &k);
      result = gathered_sum(w_homo, n);
    }
    const uint32_t bi = tile * kBatchTile + k;
    if ((gl & (G / 8 - 1)) == 0 && bi < batch) y[static_cast<size_t>(bi) * n_row + row] = result;
  }
}

// grid = (workgroups striding the rows, tiles of 8 event vectors)
template <typename F, bool HETER, bool LDS_MASK>
__global__ __launch_bounds__(1024) void csr_gather_batched_kernel(const F *__restrict__ data,
                                                                  const uint32_t *__restrict__ indices,
                                                                  const uint32_t *__restrict__ indptr,
                                                                  const uint8_t *__restrict__ masks,
                                                                  F *__restrict__ y, uint32_t n_row,
                                                                  uint32_t mask_stride, uint32_t batch) {
  extern __shared__ __attribute__((aligned(16))) unsigned char s_mask[];
  __shared__ __attribute__((aligned(16))) BatchTables s_tab;
  const uint32_t tile = blockIdx.y;
  const uint8_t *mask = masks + static_cast<size_t>(tile) * mask_stride;
  fill_batch_tables(&s_tab);
  if (LDS_MASK) {
    // rows of `masks` are padded to 16 bytes, so whole 16-byte pieces can be copied
    const uint32_t vecs = mask_stride / 16u;
    for (uint32_t i = threadIdx.x; i < vecs; i += blockDim.x)
      reinterpret_cast<uint4 *>(s_mask)[i] = reinterpret_cast<const uint4 *>(mask)[i];
  }
  __syncthreads();
  const uint8_t *probe = LDS_MASK ? reinterpret_cast<const uint8_t *>(s_mask) : mask;
  const uint32_t nnz = indptr[n_row];
  if (nnz == 0) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n_row; i += gridDim.x * blockDim.x)
      for (uint32_t k = 0; k < kBatchTile; ++k)
        if (tile * kBatchTile + k < batch) y[static_cast<size_t>(tile * kBatchTile + k) * n_row + i] = F(0);
    return;
  }
  const uint32_t mean = nnz / n_row;
  if (mean >= 32) gather_rows_batched<F, HETER, LDS_MASK, 64, 8>(data, indices, indptr, probe, y, n_row, batch, tile, &s_tab);
  else gather_rows_batched<F, HETER, LDS_MASK, 8, 2>(data, indices, indptr, probe, y, n_row, batch, tile, &s_tab);
}

template <typename F, bool HETER, bool LDS_MASK>
bool launch_gather_batched_impl(const char *target, hipStream_t stream, const F *data, const uint32_t *indices,
                                const uint32_t *indptr, const uint8_t *masks, F *y, uint32_t n_row,
                                uint32_t mask_stride, uint32_t batch, size_t lds_bytes) {
  auto kernel = csr_gather_batched_kernel<F, HETER, LDS_MASK>;
  const int block = (n_row >= 16384) ? 1024 : 256;
  if (lds_bytes > 64 * 1024) {
    static thread_local size_t attr_set_for = 0;
    if (attr_set_for < lds_bytes) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds_bytes)) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      attr_set_for = lds_bytes;
    }
  }
  int per_cu = 1;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kernel), block,
                                                   lds_bytes) != hipSuccess || per_cu < 1) {
    (void)hipGetLastError();
    per_cu = 1;
  }
  const unsigned tiles = div_up(batch, kBatchTile);
  const unsigned resident = static_cast<unsigned>(device_info().num_cu) * static_cast<unsigned>(per_cu);
  const unsigned needed = div_up(n_row, block / kWave);
  const unsigned gx = needed < resident ? (needed ? needed : 1u) : resident;
  hipLaunchKernelGGL(kernel, dim3(gx, tiles), dim3(block), lds_bytes, stream, data, indices, indptr, masks, y, n_row,
                     mask_stride, batch);
  return check_launch(target);
}

// event_csr_matvec_batching: buffers = [values, indices, indptr, events, out], every operand
// with a leading batch dimension that is indexed `bi % dim` as in the reference's CPU kernel.
template <typename F, typename VT, bool HETER>
void event_csr_batching_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque,
                              size_t opaque_len) {
  bpl_event_csr_batching_descriptor d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  if (d.batch_size == 0) return;
  if (d.values_batch == 0 || d.indices_batch == 0 || d.indptr_batch == 0 || d.events_batch == 0) {
    set_error("%s: operand batch dimensions must be at least 1", target);
    return;
  }
  const F *values = static_cast<const F *>(buffers[0]);
  const uint32_t *indices = static_cast<const uint32_t *>(buffers[1]);
  const uint32_t *indptr = static_cast<const uint32_t *>(buffers[2]);
  const VT *events = static_cast<const VT *>(buffers[3]);
  F *out = static_cast<F *>(buffers[4]);
  const uint32_t n_in = d.transpose ? d.n_row : d.n_col;
  const uint32_t n_out = d.transpose ? d.n_col : d.n_row;
  if (n_out == 0) return;
  const size_t value_stride = HETER ? d.nnz : 1u;
  const bool shared_matrix = d.values_batch == 1 && d.indices_batch == 1 && d.indptr_batch == 1;
  if (!d.transpose && shared_matrix && d.batch_size > 1 && d.n_col > 0) {
    const unsigned tiles = div_up(d.batch_size, kBatchTile);
    const uint32_t stride = div_up(d.n_col, 16) * 16u;  // the padding is never probed (columns < n_col)
    uint8_t *masks = static_cast<uint8_t *>(stream_workspace(stream, static_cast<size_t>(tiles) * stride));
    if (masks == nullptr) return;
    hipLaunchKernelGGL(pack_event_masks_kernel<VT>, dim3(div_up(d.n_col, 256), tiles), dim3(256), 0, stream, events,
                       masks, d.n_col, stride, d.batch_size, d.events_batch);
    const size_t lds_bytes = stride;
    const size_t lds_cap = kLdsBitmapCap - 2048;  // (the kernel's tables take 1.6 KB of static LDS beside the masks)
    if (lds_bytes <= lds_cap &&
        launch_gather_batched_impl<F, HETER, true>(target, stream, values, indices, indptr, masks, out, d.n_row,
                                                   stride, d.batch_size, lds_bytes))
      return;
    bpl_clear_error();
    launch_gather_batched_impl<F, HETER, false>(target, stream, values, indices, indptr, masks, out, d.n_row, stride,
                                                d.batch_size, 0);
    return;
  }
  // Transposed, one matrix for all entries: groups of up to 8 entries go through ONE sorted scatter
  // over a virtual output of group * n_col columns (entry g's columns shifted by g * n_col), fed by
  // one list of the active rows of the group's entries.  (Larger groups gain nothing more and
  // overflow the runs of the sort sooner.)
  if (d.transpose && shared_matrix && d.batch_size > 1 && d.n_row > 0 && d.n_col > 0) {
    uint32_t group = d.batch_size < 8 ? d.batch_size : 8;
    while (group > 1 && (static_cast<uint64_t>(group) * d.n_col >= (1ull << 24) ||
                         static_cast<uint64_t>(group) * d.n_row >= (1ull << 31)))
      --group;
    const uint32_t vcols = group * d.n_col;
    if (group > 1 && vcols > 8192 && bin_event_scatter_usable<F>(vcols)) {
      auto round_up = [](size_t v) { return (v + 255) / 256 * 256; };
      const size_t vrows = static_cast<size_t>(group) * d.n_row;
      const size_t list_sz = round_up(vrows * sizeof(uint2));
      const size_t base_sz = round_up(vrows * sizeof(uint32_t));
      const size_t scratch_bytes = bin_event_scatter_bytes<F>(d.n_row, vcols);
      unsigned char *ws = static_cast<unsigned char *>(stream_workspace(stream, list_sz + base_sz + scratch_bytes));
      uint32_t *counters = ws ? stream_counters(stream) : nullptr;
      if (ws != nullptr && counters != nullptr) {
        uint2 *list = reinterpret_cast<uint2 *>(ws);
        uint32_t *colbase = reinterpret_cast<uint32_t *>(ws + list_sz);
        unsigned char *scratch = ws + list_sz + base_sz;
        for (uint32_t b0 = 0; b0 < d.batch_size; b0 += group) {
          const uint32_t g = (d.batch_size - b0 < group) ? d.batch_size - b0 : group;
          // entry b0 + i reads event vector (b0 + i) % events_batch: hand the kernel the rotation
          F *o = out + static_cast<size_t>(b0) * d.n_col;
          hipLaunchKernelGGL((collect_active_rows_batched_kernel<F, VT>),
                             dim3(div_up(static_cast<uint64_t>(g) * d.n_row, 8 * kWinThreads)), dim3(kWinThreads), 0,
                             stream, indptr, events, d.n_row, d.n_col, g, d.events_batch, b0, counters, list, colbase,
                             reinterpret_cast<uint32_t *>(scratch),
                             static_cast<uint32_t>(kBinEventFillBytes / sizeof(uint32_t)), o,
                             static_cast<uint64_t>(g) * d.n_col);
          if (!bin_event_scatter<F>(stream, values, HETER, indices, indptr, o, d.n_row, g * d.n_col, counters, list,
                                    static_cast<uint32_t>(vrows), scratch, scratch_bytes, colbase)) {
            set_error("%s: the sorted scatter could not be enqueued", target);
            return;
          }
        }
        check_launch(target);
        return;
      }
      if (scratch_refused_by_capture()) return ensure_error(target, "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");
      bpl_clear_error();
    }
  }
  for (uint32_t bi = 0; bi < d.batch_size; ++bi) {
    const F *v = values + static_cast<size_t>(bi % d.values_batch) * value_stride;
    const uint32_t *ix = indices + static_cast<size_t>(bi % d.indices_batch) * d.nnz;
    const uint32_t *ip = indptr + static_cast<size_t>(bi % d.indptr_batch) * (static_cast<size_t>(d.n_row) + 1u);
    const VT *ev = events + static_cast<size_t>(bi % d.events_batch) * n_in;
    F *o = out + static_cast<size_t>(bi) * n_out;
    if (d.transpose) {
      launch_scatter<F, VT, HETER, kEvent>(ScratchSource{stream}, v, ix, ip, ev, o, d.n_row, d.n_col);
      if (!check_launch(target)) return;
    } else {
      launch_gather<F, VT, HETER, kEvent>(target, ScratchSource{stream}, v, ix, ip, ev, o, d.n_row, d.n_col);
    }
  }
}

// gpu_csr_event_sum_*_i32 (lib/gpu_event_sum.cu:48-118): the event scatter under its older name
// and buffer order, buffers = [events, indices, indptr, values, result].
template <typename F, bool HETER>
void csr_event_sum_i32_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque,
                             size_t opaque_len) {
  bpl_csr_event_sum_descriptor d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  launch_scatter<F, uint8_t, HETER, kEvent>(ScratchSource{stream}, static_cast<const F *>(buffers[3]),
                                            static_cast<const uint32_t *>(buffers[1]),
                                            static_cast<const uint32_t *>(buffers[2]),
                                            static_cast<const uint8_t *>(buffers[0]), static_cast<F *>(buffers[4]),
                                            d.pre_size, d.post_size);
  check_launch(target);
}

}  // namespace

// csr_event_sum with 64-bit index arrays (the older operator family, compat_ops.hip) through the sorted event
// scatter: the kernels read the 64-bit offsets and columns where they lie (no narrowed copy: that would move
// twelve bytes per nonzero of the whole matrix, the scatter only touches the active rows).  For results of
// more than 8,192 elements; `result` need not be zeroed.  A matrix of 2^32 nonzeros or more leaves the result
// at zero (the caller follows with its atomic kernel, which runs in that case only).  1: enqueued; 0: nothing
// enqueued, the caller takes its own path; -1: nothing enqueued and the call must fail with the error that stands.
template <typename F, bool HETER>
int csr_event_sum_wide(const char *target, hipStream_t stream, const uint8_t *events, const uint64_t *indices,
                        const uint64_t *indptr, const F *values, F *result, uint32_t pre_size, uint32_t post_size) {
  if (post_size <= 8192 || !bin_event_scatter_usable<F>(post_size)) return 0;
  auto round_up = [](size_t v) { return (v + 255) / 256 * 256; };
  const size_t list_sz = round_up(static_cast<size_t>(pre_size) * sizeof(uint2));
  const ScratchSource src{stream};
  size_t got = 0;
  unsigned char *ws = static_cast<unsigned char *>(src.request(list_sz + bin_event_scatter_bytes<F>(pre_size, post_size),
                                                               list_sz + bin_event_scatter_min_bytes<F>(post_size), &got));
  uint32_t *counters = ws ? src.counters() : nullptr;
  if (ws == nullptr || counters == nullptr) {
    if (src.failure_is_final()) {
      ensure_error(target, "nothing was enqueued: no scratch memory while the stream is being captured");
      return -1;  // (the error stands: the caller must not record a slower path into the graph)
    }
    bpl_clear_error();
    return 0;
  }
  uint2 *active_list = reinterpret_cast<uint2 *>(ws);
  const unsigned collectors = collect_workgroups<F, uint8_t, kEvent>(pre_size);
  const bool fold_zero = post_size <= 32ull * collectors * kWinThreads;
  if (!fold_zero) fill_zero(stream, result, post_size);
  launch_collect<F, uint8_t, kEvent, uint64_t>(stream, indptr, events, pre_size, counters, active_list,
                                               static_cast<F *>(nullptr), kAlways, reinterpret_cast<uint32_t *>(ws + list_sz),
                                               static_cast<uint32_t>(kBinEventFillBytes / sizeof(uint32_t)), result,
                                               fold_zero ? post_size : 0u);
  if (bin_event_scatter<F>(stream, values, HETER, indices, indptr, result, pre_size, post_size, counters, active_list,
                           pre_size, ws + list_sz, got - list_sz))
    return check_launch(target) ? 1 : -1;
  // (the sort could not run: the list is not used; the result is zero, as the caller's own kernel expects it)
  fill_zero(stream, counters, 1u);
  return 0;
}
template int csr_event_sum_wide<float, false>(const char *, hipStream_t, const uint8_t *, const uint64_t *, const uint64_t *,
                                               const float *, float *, uint32_t, uint32_t);
template int csr_event_sum_wide<float, true>(const char *, hipStream_t, const uint8_t *, const uint64_t *, const uint64_t *,
                                              const float *, float *, uint32_t, uint32_t);
template int csr_event_sum_wide<double, false>(const char *, hipStream_t, const uint8_t *, const uint64_t *, const uint64_t *,
                                                const double *, double *, uint32_t, uint32_t);
template int csr_event_sum_wide<double, true>(const char *, hipStream_t, const uint8_t *, const uint64_t *, const uint64_t *,
                                               const double *, double *, uint32_t, uint32_t);
}  // namespace bpl

// ------------------------------------------------------------------------------------------------
// Allocation-free entry point
// ------------------------------------------------------------------------------------------------
// event_csr_matvec_heter_float_bool for callers that cannot allocate device memory (code under HIP
// graph capture, serving loops, harnesses that forbid hipMalloc): the scratch memory of the call
// (stream counters, the list of active rows, fill counters and runs of the sorted scatter, partial
// outputs of the window scatter, packed event bitmaps) lives in this file-scope device array
// instead of the cached allocation.  Every GPU the library runs on holds its own copy of the array,
// at its own address, until the process ends; all calls on a GPU share it, so calls that overlap
// on one GPU (different streams) race.  It keeps the last call's contents: the launchers zero the
// counters they use before the first kernel that reads them.
namespace bpl {
namespace {
constexpr size_t kStaticScratchBytes = static_cast<size_t>(64) << 20;  // 64 MiB of arena behind the counters
}  // namespace
}  // namespace bpl

static __device__ __align__(256) unsigned char scratch[bpl::kStreamCounterBytes + bpl::kStaticScratchBytes];

namespace bpl {
namespace {
// Device address of `scratch` on the current device, looked up once per device.  (In host code the
// array's name is a stand-in for the symbol, not a device address: only this pointer may be handed to
// kernels.)  The kernels run on the device that owns `stream`; the symbol is looked up on the current
// device: a stream of another device than the current one is refused.
unsigned char *static_scratch(const char *target, hipStream_t stream) {
  constexpr int kMaxDev = 64;
  static unsigned char *ptrs[kMaxDev] = {};
  static std::mutex mu;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) {
    (void)hipGetLastError();
    set_error("%s: no current device", target);
    return nullptr;
  }
  if (stream != nullptr) {
    hipDevice_t owner = dev;
    if (hipStreamGetDevice(stream, &owner) != hipSuccess) {
      (void)hipGetLastError();
    } else if (static_cast<int>(owner) != dev) {
      set_error("%s: the stream belongs to device %d and device %d is current: make the stream's device current",
                target, static_cast<int>(owner), dev);
      return nullptr;
    }
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      set_error("%s: hipGetSymbolAddress of the static scratch array failed on device %d: %s", target, dev,
                hipGetErrorString(e));
      return nullptr;
    }
    ptrs[dev] = static_cast<unsigned char *>(p);
  }
  return ptrs[dev];
}
}  // namespace
}  // namespace bpl

extern "C" void event_csr_matvec_heter_float_bool_noalloc(bpl_stream_t stream, void **buffers, const char *opaque,
                                                          size_t opaque_len) {
  // (a malformed call is refused before the device is touched)
  bpl_twouint_onebool_descriptor d;
  if (!bpl::unpack(__func__, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    bpl::set_error("%s: null buffer table", __func__);
    return;
  }
  unsigned char *base = bpl::static_scratch(__func__, static_cast<hipStream_t>(stream));
  if (base == nullptr) return;
  bpl::ScratchSource src;
  src.stream = static_cast<hipStream_t>(stream);
  src.arena_counters = reinterpret_cast<uint32_t *>(base);
  src.arena = base + bpl::kStreamCounterBytes;
  src.arena_bytes = bpl::kStaticScratchBytes;
  bpl::event_csr_matvec_entry<float, uint8_t, true>(__func__, src, buffers, opaque, opaque_len);
}

using bpl::csr_event_sum_i32_entry;
using bpl::csr_matvec_entry;
using bpl::event_csr_batching_entry;
using bpl::event_csr_matvec_entry;

#define BPL_DEFINE(name, call)                                                                   \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    hipStream_t s = static_cast<hipStream_t>(stream);                                            \
    call;                                                                                        \
  }

// bool events are read as bytes: any nonzero byte is an event
BPL_DEFINE(event_csr_matvec_heter_float_bool, (event_csr_matvec_entry<float, uint8_t, true>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_heter_float_float, (event_csr_matvec_entry<float, float, true>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_heter_double_bool, (event_csr_matvec_entry<double, uint8_t, true>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_heter_double_double, (event_csr_matvec_entry<double, double, true>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_homo_float_bool, (event_csr_matvec_entry<float, uint8_t, false>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_homo_float_float, (event_csr_matvec_entry<float, float, false>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_homo_double_bool, (event_csr_matvec_entry<double, uint8_t, false>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_homo_double_double, (event_csr_matvec_entry<double, double, false>(__func__, bpl::ScratchSource{s}, buffers, opaque, opaque_len)))

BPL_DEFINE(csr_matvec_heter_scalar_float, (csr_matvec_entry<float, true, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_heter_scalar_double, (csr_matvec_entry<double, true, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_heter_vector_float, (csr_matvec_entry<float, true, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_heter_vector_double, (csr_matvec_entry<double, true, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_heter_adaptive_float, (csr_matvec_entry<float, true, false>(__func__, s, buffers, opaque, opaque_len, 4)))
BPL_DEFINE(csr_matvec_heter_adaptive_double, (csr_matvec_entry<double, true, false>(__func__, s, buffers, opaque, opaque_len, 4)))
BPL_DEFINE(csr_matvec_homo_scalar_float, (csr_matvec_entry<float, false, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_homo_scalar_double, (csr_matvec_entry<double, false, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_homo_vector_float, (csr_matvec_entry<float, false, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_homo_vector_double, (csr_matvec_entry<double, false, false>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_homo_adaptive_float, (csr_matvec_entry<float, false, false>(__func__, s, buffers, opaque, opaque_len, 4)))
BPL_DEFINE(csr_matvec_homo_adaptive_double, (csr_matvec_entry<double, false, false>(__func__, s, buffers, opaque, opaque_len, 4)))

BPL_DEFINE(csr_matvec_transpose_heter_float, (csr_matvec_entry<float, true, true>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_transpose_heter_double, (csr_matvec_entry<double, true, true>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_transpose_homo_float, (csr_matvec_entry<float, false, true>(__func__, s, buffers, opaque, opaque_len, 3)))
BPL_DEFINE(csr_matvec_transpose_homo_double, (csr_matvec_entry<double, false, true>(__func__, s, buffers, opaque, opaque_len, 3)))

BPL_DEFINE(event_csr_matvec_batching_heter_float_bool, (event_csr_batching_entry<float, uint8_t, true>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_heter_float_float, (event_csr_batching_entry<float, float, true>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_heter_double_bool, (event_csr_batching_entry<double, uint8_t, true>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_heter_double_double, (event_csr_batching_entry<double, double, true>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_homo_float_bool, (event_csr_batching_entry<float, uint8_t, false>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_homo_float_float, (event_csr_batching_entry<float, float, false>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_homo_double_bool, (event_csr_batching_entry<double, uint8_t, false>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(event_csr_matvec_batching_homo_double_double, (event_csr_batching_entry<double, double, false>(__func__, s, buffers, opaque, opaque_len)))

BPL_DEFINE(gpu_csr_event_sum_homo_f32_i32, (csr_event_sum_i32_entry<float, false>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(gpu_csr_event_sum_homo_f64_i32, (csr_event_sum_i32_entry<double, false>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(gpu_csr_event_sum_heter_f32_i32, (csr_event_sum_i32_entry<float, true>(__func__, s, buffers, opaque, opaque_len)))
BPL_DEFINE(gpu_csr_event_sum_heter_f64_i32, (csr_event_sum_i32_entry<double, true>(__func__, s, buffers, opaque, opaque_len)))
