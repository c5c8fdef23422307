// event_info ("nonzero"): ordered compaction of the nonzero positions of an event vector.
//
//   buffers = [events T[batch][size], event_ids int32[batch][size], event_num int32[batch]]
//   opaque  = bpl_nonzero_descriptor {event_size, batch_size}
//   event_ids[b] = positions i with events[b][i] != 0 in increasing order, then -1 up to `size`;
//   event_num[b] = their number.
//
// The reference's CPU kernel produces exactly this (brainpylib/_src/event_ops/
// event_info_collection.py:143-155); its GPU kernel fills the same set in arbitrary order
// (lib/gpu_event_info.cu:11-45), so the ordered result satisfies both.
//
// Three passes over tiles of 4,096 elements (256 threads x 16 elements, element e * 256 + t of the
// tile by thread t, so that every load is contiguous across the wave and 16 of them are in
// flight): per-tile counts (ballot + popcount); an exclusive scan of the tile counts of each
// batch row by one workgroup; then every tile re-derives its flags, ranks its events (wave
// masks, a 64-entry scan over (sub-row, wave) counts), lists them in LDS and writes two
// contiguous runs: its events at their ranks and its share of the -1 tail.
//
// Reference boundary: lib/gpu_event_info.cu:48-96 (buffers, descriptor, target names).
#include "common.h"
#include "targets.h"

namespace bpl {
namespace {

constexpr int kScanThreads = 1024;  // the scan kernel's workgroup
constexpr int kThreads = 256;
constexpr int kPerThread = 16;
constexpr uint32_t kTile = kThreads * kPerThread;
constexpr int kWavesPerTile = kThreads / kWave;
static_assert(kPerThread * kWavesPerTile == kWave, "one wave scans the (sub-row, wave) counts");

// wave masks of the tile's 16 sub-rows of 256 elements: m[e] covers elements e * 256 + wave * 64 + lane
template <typename T>
__device__ __forceinline__ void tile_masks(const T *__restrict__ row, uint32_t size, uint32_t tile_start,
                                           uint64_t (&m)[kPerThread]) {
  T v[kPerThread];
#pragma unroll
  for (int e = 0; e < kPerThread; ++e) {
    const uint32_t i = tile_start + e * kThreads + threadIdx.x;
    v[e] = i < size ? row[i] : T(0);
  }
#pragma unroll
  for (int e = 0; e < kPerThread; ++e) m[e] = __ballot(v[e] != T(0));
}

// One-byte events, tile start aligned to 16 bytes: thread t takes the 16 consecutive bytes
// 16 t .. 16 t + 15 of the tile with one load; bit i of the result = byte i is nonzero.
__device__ __forceinline__ uint32_t byte_flags16(const uint8_t *__restrict__ row, uint32_t size, uint32_t tile_start) {
  const uint32_t i0 = tile_start + 16u * threadIdx.x;
  if (i0 + 16u <= size) {
    const uint4 q = *reinterpret_cast<const uint4 *>(row + i0);
    return nonzero_bytes_nibble(q.x) | (nonzero_bytes_nibble(q.y) << 4) | (nonzero_bytes_nibble(q.z) << 8) |
           (nonzero_bytes_nibble(q.w) << 12);
  }
  uint32_t f = 0;
  for (uint32_t i = 0; i < 16u; ++i)
    if (i0 + i < size && row[i0 + i] != 0) f |= 1u << i;
  return f;
}

template <typename T>
__device__ __forceinline__ bool bytes_aligned(const T *row, uint32_t tile_start) {
  return sizeof(T) == 1 && ((reinterpret_cast<uintptr_t>(row) + tile_start) & 15u) == 0;
}

// counts[b][tile] = number of events in the tile
template <typename T>
__global__ __launch_bounds__(kThreads) void tile_count_kernel(const T *__restrict__ ev, uint32_t size, uint32_t n_tiles,
                                                             uint32_t *__restrict__ counts) {
  __shared__ uint32_t s_cnt[kWavesPerTile];
  const uint32_t b = blockIdx.y, tile = blockIdx.x;
  const T *row = ev + static_cast<size_t>(b) * size;
  uint32_t c = 0;
  if (bytes_aligned(row, tile * kTile)) {
    c = wave_sum(static_cast<uint32_t>(__popc(byte_flags16(reinterpret_cast<const uint8_t *>(row), size, tile * kTile))));
  } else {
    uint64_t m[kPerThread];
    tile_masks(row, size, tile * kTile, m);
#pragma unroll
    for (int e = 0; e < kPerThread; ++e) c += static_cast<uint32_t>(__popcll(m[e]));
  }
  if (lane_id() == 0) s_cnt[threadIdx.x / kWave] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kWavesPerTile; ++w) t += s_cnt[w];
    counts[static_cast<size_t>(b) * n_tiles + tile] = t;
  }
}

// in place: counts[b][*] -> exclusive prefix; event_num[b] = total.  One workgroup per batch row.
__global__ __launch_bounds__(kScanThreads) void tile_scan_kernel(uint32_t *__restrict__ counts, uint32_t n_tiles,
                                                                int32_t *__restrict__ event_num) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  __shared__ uint32_t s_carry;
  uint32_t *row = counts + static_cast<size_t>(blockIdx.x) * n_tiles;
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wave = threadIdx.x / kWave;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (uint32_t base = 0; base < n_tiles; base += kScanThreads) {
    const uint32_t i = base + threadIdx.x;
    const uint32_t v = i < n_tiles ? row[i] : 0u;
    const uint32_t incl = wave_inclusive_scan_u32(v);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = s_carry;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave[w];
    if (i < n_tiles) row[i] = before + incl - v;
    __syncthreads();
    if (threadIdx.x == kScanThreads - 1) s_carry = before + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) event_num[blockIdx.x] = static_cast<int32_t>(s_carry);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void tile_write_kernel(const T *__restrict__ ev, uint32_t size, uint32_t n_tiles,
                                                             const uint32_t *__restrict__ offsets,
                                                             const int32_t *__restrict__ event_num,
                                                             int32_t *__restrict__ ids) {
  __shared__ uint32_t s_pre[kWave];    // events before (sub-row e, wave w), entry e * 4 + w
  __shared__ int32_t s_list[kTile];    // the tile's event positions in order
  __shared__ uint32_t s_total;
  const uint32_t b = blockIdx.y, tile = blockIdx.x;
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wave = threadIdx.x / kWave;
  const uint32_t tile_start = tile * kTile;
  const T *row = ev + static_cast<size_t>(b) * size;
  if (bytes_aligned(row, tile_start)) {
    // thread t holds elements 16 t .. 16 t + 15: ranks follow the thread order
    uint32_t f = byte_flags16(reinterpret_cast<const uint8_t *>(row), size, tile_start);
    const uint32_t c = static_cast<uint32_t>(__popc(f));
    const uint32_t incl = wave_inclusive_scan_u32(c);
    if (lane == kWave - 1) s_pre[wave] = incl;
    __syncthreads();
    uint32_t k = incl - c;
    for (uint32_t w = 0; w < wave; ++w) k += s_pre[w];
    if (threadIdx.x == kThreads - 1) s_total = k + c;
    while (f) {
      const uint32_t bit = static_cast<uint32_t>(__ffs(static_cast<int>(f))) - 1u;
      f &= f - 1u;
      s_list[k++] = static_cast<int32_t>(tile_start + 16u * threadIdx.x + bit);
    }
  } else {
    uint64_t m[kPerThread];
    tile_masks(row, size, tile_start, m);
    if (lane == 0) {
#pragma unroll
      for (int e = 0; e < kPerThread; ++e) s_pre[e * kWavesPerTile + wave] = static_cast<uint32_t>(__popcll(m[e]));
    }
    __syncthreads();
    if (wave == 0) {
      const uint32_t c = s_pre[lane];
      const uint32_t incl = wave_inclusive_scan_u32(c);
      s_pre[lane] = incl - c;
      if (lane == kWave - 1) s_total = incl;
    }
    __syncthreads();
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int e = 0; e < kPerThread; ++e) {
      if ((m[e] >> lane) & 1ull) {
        const uint32_t k = s_pre[e * kWavesPerTile + wave] + static_cast<uint32_t>(__popcll(m[e] & below));
        s_list[k] = static_cast<int32_t>(tile_start + e * kThreads + threadIdx.x);
      }
    }
  }
  __syncthreads();
  int32_t *out = ids + static_cast<size_t>(b) * size;
  const uint32_t cnt = s_total;
  const uint32_t off = offsets[static_cast<size_t>(b) * n_tiles + tile];  // events before this tile
  for (uint32_t i = threadIdx.x; i < cnt; i += kThreads) out[off + i] = s_list[i];
  // the tile's elements that are no events account for as many -1 entries after the last event
  const uint32_t valid = (size - tile_start < kTile) ? size - tile_start : kTile;
  const uint32_t tail = static_cast<uint32_t>(event_num[b]) + (tile_start - off);
  for (uint32_t i = threadIdx.x; i < valid - cnt; i += kThreads) out[tail + i] = -1;
}

// Rows of at most one tile (4,096 elements): one WAVE per row does all of it, 64 elements a step (flags by
// ballot, ranks by the count of lower lanes), then the -1 tail and the count.  (A workgroup per row and three
// kernels, as for long rows, took 4.4 ms for 1,000,000 rows of 100.)
template <typename T>
__global__ __launch_bounds__(kThreads) void short_rows_kernel(const T *__restrict__ ev, uint32_t size, uint32_t batch,
                                                             int32_t *__restrict__ ids, int32_t *__restrict__ event_num) {
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const uint64_t below = (1ull << lane) - 1ull;
  const uint32_t waves = gridDim.x * (kThreads / kWave);
  for (uint32_t b = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave; b < batch; b += waves) {
    const T *row = ev + static_cast<size_t>(b) * size;
    int32_t *out = ids + static_cast<size_t>(b) * size;
    uint32_t n = 0;
    for (uint32_t i0 = 0; i0 < size; i0 += kWave) {
      const uint32_t i = i0 + lane;
      const bool on = i < size && row[i] != T(0);
      const uint64_t m = __ballot(on);
      if (on) out[n + static_cast<uint32_t>(__popcll(m & below))] = static_cast<int32_t>(i);
      n += static_cast<uint32_t>(__popcll(m));
    }
    for (uint32_t i = n + lane; i < size; i += kWave) out[i] = -1;
    if (lane == 0) event_num[b] = static_cast<int32_t>(n);
  }
}

template <typename T>
void nonzero_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t opaque_len) {
  bpl_nonzero_descriptor d;
  if (!unpack(target, opaque, opaque_len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  const T *ev = static_cast<const T *>(buffers[0]);
  int32_t *ids = static_cast<int32_t *>(buffers[1]);
  int32_t *num = static_cast<int32_t *>(buffers[2]);
  if (d.batch_size == 0) return;
  if (d.event_size == 0) {
    fill_zero(stream, num, d.batch_size);
    check_launch(target);
    return;
  }
  if (d.event_size <= kTile && d.batch_size >= 64) {  // many short rows: a wave each
    const uint32_t rows_per_wg = kThreads / kWave;
    uint32_t grid = div_up(d.batch_size, rows_per_wg);
    const uint32_t resident = 8u * static_cast<uint32_t>(device_info().num_cu);
    if (grid > 8u * resident) grid = 8u * resident;
    hipLaunchKernelGGL(short_rows_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, ev, d.event_size, d.batch_size, ids, num);
    check_launch(target);
    return;
  }
  const uint32_t n_tiles = div_up(d.event_size, kTile);
  // (a grid holds 65,535 batch rows in its second dimension: more rows are taken that many at a time)
  constexpr uint32_t kMaxGridY = 65535;
  const uint32_t rows_at_once = d.batch_size < kMaxGridY ? d.batch_size : kMaxGridY;
  uint32_t *counts = static_cast<uint32_t *>(
      stream_workspace(stream, static_cast<size_t>(rows_at_once) * n_tiles * sizeof(uint32_t)));
  if (counts == nullptr) return;
  for (uint32_t b0 = 0; b0 < d.batch_size; b0 += kMaxGridY) {
    const uint32_t rows = d.batch_size - b0 < kMaxGridY ? d.batch_size - b0 : kMaxGridY;
    const T *ev_b = ev + static_cast<size_t>(b0) * d.event_size;
    int32_t *ids_b = ids + static_cast<size_t>(b0) * d.event_size;
    const dim3 grid(n_tiles, rows);
    hipLaunchKernelGGL(tile_count_kernel<T>, grid, dim3(kThreads), 0, stream, ev_b, d.event_size, n_tiles, counts);
    hipLaunchKernelGGL(tile_scan_kernel, dim3(rows), dim3(kScanThreads), 0, stream, counts, n_tiles, num + b0);
    hipLaunchKernelGGL(tile_write_kernel<T>, grid, dim3(kThreads), 0, stream, ev_b, d.event_size, n_tiles, counts,
                       static_cast<const int32_t *>(num + b0), ids_b);
  }
  check_launch(target);
}

}  // namespace
}  // namespace bpl

using namespace bpl;

#define BPL_DEFINE(name, T)                                                                       \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    nonzero_entry<T>(__func__, static_cast<hipStream_t>(stream), buffers, opaque, opaque_len);      \
  }

BPL_DEFINE(nonzero_bool, uint8_t)
BPL_DEFINE(nonzero_int, int32_t)
BPL_DEFINE(nonzero_long, int64_t)
BPL_DEFINE(nonzero_float, float)
BPL_DEFINE(nonzero_double, double)
