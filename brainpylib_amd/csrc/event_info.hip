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
// Three passes over 1024-element tiles: per-tile counts (ballot + popcount), an exclusive scan
// of the tile counts of each batch row by one workgroup, then every tile re-derives its flags
// and writes its ranked positions; the tail is filled with -1 in the same pass.
//
// Reference boundary: lib/gpu_event_info.cu:48-96 (buffers, descriptor, target names).
#include "common.h"
#include "targets.h"

namespace bpl {
namespace {

constexpr int kTile = 1024;

template <typename T>
__device__ __forceinline__ bool flag_at(const T *__restrict__ ev, uint32_t size, uint32_t b, uint32_t i) {
  return i < size && ev[static_cast<size_t>(b) * size + i] != T(0);
}

// counts[b][tile] = number of events in the tile
template <typename T>
__global__ __launch_bounds__(kTile) void tile_count_kernel(const T *__restrict__ ev, uint32_t size, uint32_t n_tiles,
                                                          uint32_t *__restrict__ counts) {
  __shared__ uint32_t s_cnt[kTile / kWave];
  const uint32_t b = blockIdx.y, tile = blockIdx.x;
  const bool on = flag_at(ev, size, b, tile * kTile + threadIdx.x);
  const uint64_t m = __ballot(on);
  if (lane_id() == 0) s_cnt[threadIdx.x / kWave] = static_cast<uint32_t>(__popcll(m));
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kTile / kWave; ++w) t += s_cnt[w];
    counts[static_cast<size_t>(b) * n_tiles + tile] = t;
  }
}

// in place: counts[b][*] -> exclusive prefix; event_num[b] = total.  One workgroup per batch row.
__global__ __launch_bounds__(kTile) void tile_scan_kernel(uint32_t *__restrict__ counts, uint32_t n_tiles,
                                                         int32_t *__restrict__ event_num) {
  __shared__ uint32_t s_wave[kTile / kWave];
  __shared__ uint32_t s_carry;
  uint32_t *row = counts + static_cast<size_t>(blockIdx.x) * n_tiles;
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wave = threadIdx.x / kWave;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (uint32_t base = 0; base < n_tiles; base += kTile) {
    const uint32_t i = base + threadIdx.x;
    const uint32_t v = i < n_tiles ? row[i] : 0u;
    const uint32_t incl = wave_inclusive_scan_u32(v);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = s_carry;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave[w];
    if (i < n_tiles) row[i] = before + incl - v;
    __syncthreads();
    if (threadIdx.x == kTile - 1) s_carry = before + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) event_num[blockIdx.x] = static_cast<int32_t>(s_carry);
}

template <typename T>
__global__ __launch_bounds__(kTile) void tile_write_kernel(const T *__restrict__ ev, uint32_t size, uint32_t n_tiles,
                                                          const uint32_t *__restrict__ offsets,
                                                          const int32_t *__restrict__ event_num,
                                                          int32_t *__restrict__ ids) {
  __shared__ uint32_t s_cnt[kTile / kWave];
  const uint32_t b = blockIdx.y, tile = blockIdx.x;
  const uint32_t i = tile * kTile + threadIdx.x;
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wave = threadIdx.x / kWave;
  const bool on = flag_at(ev, size, b, i);
  const uint64_t m = __ballot(on);
  if (lane == 0) s_cnt[wave] = static_cast<uint32_t>(__popcll(m));
  __syncthreads();
  int32_t *out = ids + static_cast<size_t>(b) * size;
  if (on) {
    uint32_t pos = offsets[static_cast<size_t>(b) * n_tiles + tile];
    for (uint32_t w = 0; w < wave; ++w) pos += s_cnt[w];
    pos += static_cast<uint32_t>(__popcll(m & ((1ull << lane) - 1ull)));
    out[pos] = static_cast<int32_t>(i);
  }
  // positions at and beyond the number of events hold -1 (written by the thread of that position)
  if (i < size && i >= static_cast<uint32_t>(event_num[b])) out[i] = -1;
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
  if (d.batch_size > 65535) {
    set_error("%s: batch_size %u exceeds 65535", target, d.batch_size);
    return;
  }
  const uint32_t n_tiles = div_up(d.event_size, kTile);
  uint32_t *counts = static_cast<uint32_t *>(
      stream_workspace(stream, static_cast<size_t>(d.batch_size) * n_tiles * sizeof(uint32_t)));
  if (counts == nullptr) return;
  const dim3 grid(n_tiles, d.batch_size);
  hipLaunchKernelGGL(tile_count_kernel<T>, grid, dim3(kTile), 0, stream, ev, d.event_size, n_tiles, counts);
  hipLaunchKernelGGL(tile_scan_kernel, dim3(d.batch_size), dim3(kTile), 0, stream, counts, n_tiles, num);
  hipLaunchKernelGGL(tile_write_kernel<T>, grid, dim3(kTile), 0, stream, ev, d.event_size, n_tiles, counts, num, ids);
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
