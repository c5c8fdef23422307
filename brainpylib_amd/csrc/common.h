// Internal helpers shared by the HIP sources of libbrainpylib_amd.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstring>

#include "../../include/brainpylib_amd.h"

namespace bpl {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- error channel (host) ---------------------------------------------------------------------
void set_error(const char *fmt, ...);

// Checks `opaque_len == sizeof(T)` and copies the descriptor out of the opaque bytes
// (the pointer is not assumed to be aligned).  Returns false and records an error otherwise.
// Every entry point calls this first (through unpack): what an earlier call on this thread left in
// the capture-refusal flag says nothing about this one.
void begin_call();

template <typename T>
inline bool unpack(const char *target, const char *opaque, size_t opaque_len, T *out) {
  begin_call();
  if (opaque == nullptr || opaque_len != sizeof(T)) {
    set_error("%s: invalid opaque object size %zu (expected %zu)", target, opaque_len, sizeof(T));
    return false;
  }
  std::memcpy(out, opaque, sizeof(T));
  return true;
}

// Records a failed launch; returns true if the last launch was fine.
bool check_launch(const char *target);

// Device properties of the current device, cached per device id.
struct DeviceInfo {
  int num_cu = 0;
  int lds_per_block = 0;  // bytes of LDS one workgroup may use
};
const DeviceInfo &device_info();

// Scratch device memory for operators that need a staging buffer (the custom-call ABI provides
// none): one allocation per (device, stream), grown on demand and kept until the process ends.
// Work enqueued on one stream is ordered, so calls on the same stream can share the buffer;
// calls on different streams get different buffers.  A buffer that has been handed out is never
// freed: when a larger one is needed the old one is retired (kept allocated), because work that
// was enqueued earlier, or a HIP graph captured earlier on the stream, may still use it.  Growing
// needs hipMalloc, which cannot run while the stream is being captured into a graph: then the
// call fails (nullptr, error recorded, nothing enqueued), so every size must have been used once
// on the stream before it is captured.  nullptr (error recorded) also if the allocation fails.
void *stream_workspace(hipStream_t stream, size_t bytes);

// A few zero-initialised 32-bit counters per (device, stream).  The first one (the scatter's
// active-row count) is left at zero again by every user; the others carry nothing from call to
// call.  nullptr if the allocation fails (or would be needed during a capture).
uint32_t *stream_counters(hipStream_t stream);
constexpr size_t kStreamCounterBytes = 256;

// True if the calling thread's most recent stream_workspace() / stream_counters() call failed
// because the stream was being captured.  A launcher that would otherwise fall back to a path
// that needs less scratch memory must then give up with the error standing: a graph that
// silently records the slow path would replay it for good.
bool scratch_refused_by_capture();
// A call that gives up must leave an error: records "<target>: <why>" unless one already stands.
void ensure_error(const char *target, const char *why);

// Where the launchers of one call take their scratch memory from: the cached allocation of the
// call's stream (above), or a fixed arena that the entry point owns and that is never grown (the
// allocation-free entry point's static device array).  Either way ONE buffer serves the whole
// call: every request() of a call returns the same base address, and the launchers lay their
// sub-buffers out inside it.
struct ScratchSource {
  hipStream_t stream = nullptr;
  unsigned char *arena = nullptr;     // fixed arena (device memory), or nullptr: the cached allocation
  size_t arena_bytes = 0;
  uint32_t *arena_counters = nullptr;  // kStreamCounterBytes of device memory beside the arena

  bool fixed() const { return arena != nullptr; }
  // after a failed request(): must the call fail (true), or may it fall back to a path that needs
  // less scratch memory (an allocation failed: false)?
  bool failure_is_final() const { return fixed() || scratch_refused_by_capture(); }
  // `want` bytes if they can be had, at least `need`; *got receives the size obtained.  nullptr,
  // with an error recorded, if `need` bytes are not available.
  void *request(size_t want, size_t need, size_t *got) const;
  void *request(size_t bytes) const {
    size_t got = 0;
    return request(bytes, bytes, &got);
  }
  uint32_t *counters() const { return fixed() ? arena_counters : stream_counters(stream); }
};

// Transposed CSR times dense vector through coarse sorting of the products (csr_bin_scatter.hip),
// for outputs much wider than LDS.  `nnz` must be the matrix's nonzero count (indptr[n_row]).
// bin_scatter returns false, having enqueued nothing, if it cannot run (no scratch memory).
template <typename F>
bool bin_scatter_usable(uint32_t n_col, uint32_t nnz);
template <typename F>
bool bin_scatter(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                 const uint32_t *indptr, const F *vec, F *y, uint32_t n_row, uint32_t n_col, uint32_t nnz);

// coo_atomic_sum / coo_event_sum through windows of the result in LDS (coo_window_sum.hip): taken for a long
// connection list and a result of a few windows.  EVENT: connection i counts if
// events[pre_ids[i]] and carries values[i]; otherwise it carries values[pre_ids[i]]; HETER false: values[0].
// 1: enqueued; 0: nothing enqueued, the caller takes another path; -1: nothing enqueued and the call must fail
// with the error that stands.
template <typename F, typename I, bool HETER, bool EVENT>
int coo_window_sum(const char *target, hipStream_t stream, const uint8_t *events, const F *values, const I *post_ids,
                   const I *pre_ids, F *result, uint32_t conn_size, uint32_t post_size);
// The same sums with a weight per connection or source into a wider result, through bins (the coarse-sorted
// scatter); same return values.
template <typename F, typename I, bool EVENT>
int coo_bin_sum(const char *target, hipStream_t stream, const uint8_t *events, const F *values, const I *post_ids,
                const I *pre_ids, F *result, uint32_t conn_size, uint32_t post_size);

// Transposed CSR times dense vector for outputs of at most kFlatWindowMaxSlices windows of kFlatWindowMaxCols
// columns (a float64 window in LDS per workgroup, the workgroups of a window equal shares of the nonzeros;
// csr_bin_scatter.hip).  false, having enqueued nothing, if it cannot run (wider output, no scratch memory).
constexpr uint32_t kFlatWindowMaxCols = 16384;
constexpr uint32_t kFlatWindowMaxSlices = 2;  // (a third window costs a third pass over the matrix: sorting wins)
template <typename F>
bool flat_window_scatter(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                         const uint32_t *indptr, const F *vec, F *y, uint32_t n_row, uint32_t n_col);

// The same for event input (event_csr_matvec, transposed, wide outputs): the caller lists the
// active rows on the device, (first nonzero, length) each in `active_list`, their number in
// active_count[0] (the list has room for `list_cap` rows); `scratch` is device memory of `scratch_bytes` bytes whose first
// kBinEventFillBytes are zero; y is zeroed.  Enqueues the two kernels; the second one sets
// active_count[0] back to zero.  false (nothing enqueued) if it cannot run.
// The scratch memory behind the fill counters holds the runs of (column, weight) pairs: the call
// works with any size from bin_event_scatter_min_bytes() on (pairs that find their run full go
// through direct atomics, far more slowly), and bin_event_scatter_bytes() is the size to ask for.
// Batched calls (several event vectors, one matrix) hand in one list over all batch entries, n_col
// = batch * columns, and `active_colbase` = what to add to the columns of each listed row (its
// batch entry * columns); n_row stays the matrix's row count (indptr has n_row + 1 entries).
constexpr size_t kBinEventFillBytes = 131072;
template <typename F>
bool bin_event_scatter_usable(uint32_t n_col);
template <typename F>
size_t bin_event_scatter_bytes(uint32_t n_row, uint32_t n_col);
template <typename F>
size_t bin_event_scatter_min_bytes(uint32_t n_col);
// I: the type of the column indices and row offsets (uint32_t, or uint64_t for the older csr_event_sum; the
// listed (first nonzero, length) entries are 32-bit either way).
template <typename F, typename I>
bool bin_event_scatter(hipStream_t stream, const F *data, bool heter, const I *indices, const I *indptr,
                       F *y, uint32_t n_row, uint32_t n_col, uint32_t *active_count, const uint2 *active_list,
                       uint32_t list_cap, void *scratch, size_t scratch_bytes,
                       const uint32_t *active_colbase = nullptr);
// csr_event_sum with 64-bit index arrays through the sorted event scatter (csr_ops.hip).  1: enqueued (a matrix of
// 2^32 nonzeros or more leaves the zeroed result untouched); 0: nothing enqueued, take another path; -1: failed.
template <typename F, bool HETER>
int csr_event_sum_wide(const char *target, hipStream_t stream, const uint8_t *events, const uint64_t *indices,
                        const uint64_t *indptr, const F *values, F *result, uint32_t pre_size, uint32_t post_size);

// mt19937 states of the generator streams seed + first .. seed + first + count - 1, 624 words each, seeded on
// the vector unit, 64 streams per wave (jitconn_ops.hip).  A wave that seeds the stream it walks holds its
// CU's one scalar unit for about 2 us.
void jitconn_seed_streams(hipStream_t stream, uint32_t seed, uint32_t first, uint32_t count, uint32_t *states);

// Event input and an output of at most 8,192 columns (a homogeneous weight: of a few slices of 14,848): the listed
// active rows' nonzeros are walked flat into one window in LDS per workgroup (csr_bin_scatter.hip).  `counters`: the stream's counters, [0] the number
// of listed rows (set back to zero by the second kernel), [1] used between the two kernels.  `scratch`:
// window_event_scatter_bytes() of device memory.  y need not be zeroed.  false (nothing enqueued) if it
// cannot run.
template <typename F>
bool window_event_scatter_usable(uint32_t n_row, uint32_t n_col, bool heter);
template <typename F>
size_t window_event_scatter_bytes(uint32_t n_col);
template <typename F>
bool window_event_scatter(hipStream_t stream, const F *data, bool heter, const uint32_t *indices, const uint32_t *indptr,
                          F *y, uint32_t n_row, uint32_t n_col, uint32_t *counters, const uint2 *active_list,
                          uint32_t list_cap, void *scratch, size_t scratch_bytes, const void *events = nullptr,
                          uint32_t event_width = 0);
// With `events` (the events themselves, elements of event_width = 1, 4 or 8 bytes: bytes, float or double, nonzero =
// event) the kernel finds the active rows itself: no list (active_list may be nullptr, list_cap is not used), one
// launch fewer.  For at most 32,768 rows; the output may then have up to 14,848 columns (taken in two slices;
// with a homogeneous weight up to 59,392 in four).
bool window_event_scatter_self_usable(uint32_t n_row, uint32_t n_col, bool heter);

// Second half of the coarse-sorted scatter for producers other than the CSR one: adds bins laid
// out uniformly, bin (p, b) = the places from (p * n_win + b) * cap with counts[b * producers + p]
// entries (counts above cap mean cap), n_win = ceil(n_out / 2^shift), into the zeroed y.  The places are
// BinPair<F> entries (bins.h), or, `packed` (windows of at most 2^16 outputs, cap a multiple of 4): an
// array of producers * n_win * cap values with the 16-bit positions within the window in an array behind
// it.  `reset` (optional): a device counter of the producer's that the kernel sets to zero.
template <typename F>
bool add_uniform_bins(const char *target, hipStream_t stream, F *y, uint32_t n_out, uint32_t shift, uint32_t producers,
                      uint32_t cap, const void *pairs, bool packed, const uint32_t *counts, uint32_t *reset);

inline unsigned div_up(unsigned long long a, unsigned long long b) {
  return static_cast<unsigned>((a + b - 1) / b);
}

// ---- zero fill on the stream (a kernel, not a memset node, so that the call sequence can be
// captured into a HIP graph) ---------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void fill_zero_kernel(T *__restrict__ p, uint32_t n) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < n) p[i] = T(0);
}

template <typename T>
inline void fill_zero(hipStream_t stream, T *p, uint32_t n) {
  if (n == 0) return;
  hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(div_up(n, 256)), dim3(256), 0, stream, p, n);
}

// ---- device helpers -----------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }

// events are `bool` (one byte, any nonzero byte counts) or a float type (nonzero, NaN included).
template <typename VT>
__device__ __forceinline__ bool is_event(VT v) {
  return v != VT(0);
}

// Sum over the 64 lanes of a wave; every lane receives the total.
template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Sum over aligned groups of G consecutive lanes (G a power of two <= 64).
template <int G, typename T>
__device__ __forceinline__ T group_sum(T v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Inclusive prefix sum of a 32-bit value across the wave (wrapping), via DPP row shifts and
// row broadcasts.
__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v) {
  int x = static_cast<int>(v);
  // within each row of 16 lanes
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
  // carry row totals: lane 15 of rows 0,2 into rows 1,3; then lane 31 into rows 2,3
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return static_cast<uint32_t>(x);
}

// Bits [0,32) = events[base + b] != 0, zero beyond n.
template <typename VT>
__device__ __forceinline__ uint32_t pack_events32(const VT *__restrict__ ev, uint32_t base, uint32_t n) {
  uint32_t m = 0;
  for (uint32_t b = 0; b < 32; ++b) {
    const uint32_t i = base + b;
    if (i < n && is_event(ev[i])) m |= 1u << b;
  }
  return m;
}

// 4 nonzero-byte flags of a dword, gathered into the low nibble.
__device__ __forceinline__ uint32_t nonzero_bytes_nibble(uint32_t v) {
  const uint32_t nz = (((v & 0x7f7f7f7fu) + 0x7f7f7f7fu) | v) & 0x80808080u;
  // bit 7,15,23,31 -> bits 24..27 of the product (the partial products never collide)
  return (((nz >> 7) * 0x01020408u) >> 24) & 0xfu;
}

template <>
__device__ __forceinline__ uint32_t pack_events32<uint8_t>(const uint8_t *__restrict__ ev, uint32_t base,
                                                            uint32_t n) {
  const uint8_t *p = ev + base;
  if (base + 32 <= n && (reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
    const uint4 a = *reinterpret_cast<const uint4 *>(p);
    const uint4 b = *reinterpret_cast<const uint4 *>(p + 16);
    return nonzero_bytes_nibble(a.x) | (nonzero_bytes_nibble(a.y) << 4) | (nonzero_bytes_nibble(a.z) << 8) |
           (nonzero_bytes_nibble(a.w) << 12) | (nonzero_bytes_nibble(b.x) << 16) |
           (nonzero_bytes_nibble(b.y) << 20) | (nonzero_bytes_nibble(b.z) << 24) |
           (nonzero_bytes_nibble(b.w) << 28);
  }
  uint32_t m = 0;
  for (uint32_t b = 0; b < 32; ++b) {
    const uint32_t i = base + b;
    if (i < n && ev[i] != 0) m |= 1u << b;
  }
  return m;
}

// An event vector already packed to one bit per element (32 per word), by pack_event_bitmap().
struct PackedBits {
  uint32_t w;
  // (never evaluated: only to let the dense-vector branches of the shared kernels compile)
  __host__ __device__ explicit operator float() const { return 0.f; }
  __host__ __device__ explicit operator double() const { return 0.0; }
};
template <>
__device__ __forceinline__ bool is_event<PackedBits>(PackedBits v) {
  return v.w != 0u;
}
template <>
__device__ __forceinline__ uint32_t pack_events32<PackedBits>(const PackedBits *__restrict__ ev, uint32_t base,
                                                               uint32_t n) {
  return ev[base >> 5].w;  // base is a multiple of 32; bits beyond n are zero
}

// Is element i of the event vector set?
template <typename VT>
__device__ __forceinline__ bool probe_event(const VT *__restrict__ ev, uint32_t i) {
  return is_event(ev[i]);
}
template <>
__device__ __forceinline__ bool probe_event<PackedBits>(const PackedBits *__restrict__ ev, uint32_t i) {
  return (ev[i >> 5].w >> (i & 31u)) & 1u;
}

// bits[w] bit b = ev[32 w + b] != 0 (zero beyond n): coalesced loads, one ballot per 64 elements.
template <typename VT>
__global__ __launch_bounds__(256) void pack_event_bitmap_kernel(const VT *__restrict__ ev, uint32_t n,
                                                                uint32_t *__restrict__ bits) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t waves = gridDim.x * (256 / kWave);
  const uint32_t groups = (n + kWave - 1) / kWave;
  for (uint32_t g = blockIdx.x * (256 / kWave) + threadIdx.x / kWave; g < groups; g += waves) {
    const uint32_t i = g * kWave + lane;
    const unsigned long long m = __ballot(i < n && is_event(ev[i]));
    if (lane == 0) bits[2 * g] = static_cast<uint32_t>(m);
    if (lane == 32 && 2 * g + 1 < (n + 31) / 32) bits[2 * g + 1] = static_cast<uint32_t>(m >> 32);
  }
}

// Two-level bitmap for event vectors whose bitmap does not fit LDS.  Behind the exact bitmap
// (ceil(n / 32) words, padded to coarse_offset_words(n)) sits a coarse one: bit c = any of the
// elements [c << g, (c + 1) << g) is set, with g = coarse_shift(n) the smallest shift for which
// the coarse bitmap fits kLdsBitmapCap bytes.  A kernel keeps the coarse bitmap in LDS and looks
// at the exact one, in global memory, only where the coarse bit is set.
constexpr uint32_t kLdsBitmapCap = 160u * 1024u - 1024u;
__host__ __device__ inline uint32_t coarse_bits(uint32_t n, uint32_t g) { return n ? ((n - 1u) >> g) + 1u : 0u; }
__host__ __device__ inline uint32_t coarse_shift(uint32_t n, uint32_t cap_bytes = kLdsBitmapCap) {
  uint32_t g = 0;
  while ((coarse_bits(n, g) + 31u) / 32u * 4u > cap_bytes) ++g;
  return g;
}
__host__ __device__ inline uint32_t coarse_offset_words(uint32_t n) { return ((n + 31u) / 32u + 63u) / 64u * 64u; }

static __global__ __launch_bounds__(256) void coarsen_bitmap_kernel(const uint32_t *__restrict__ bits, uint32_t n_words,
                                                             uint32_t g, uint32_t *__restrict__ coarse,
                                                             uint32_t n_coarse_words) {
  const uint32_t w = blockIdx.x * 256u + threadIdx.x;
  if (w >= n_coarse_words) return;
  uint32_t out = 0;
  for (uint32_t i = 0; i < 32u; ++i) {
    const uint64_t c = static_cast<uint64_t>(w) * 32u + i;
    uint32_t any = 0;
    if (g >= 5u) {
      const uint64_t first = c << (g - 5u);
      for (uint64_t k = 0; k < (1ull << (g - 5u)) && first + k < n_words; ++k) any |= bits[first + k];
    } else {
      const uint64_t word = c >> (5u - g);
      const uint32_t sub = static_cast<uint32_t>(c) & ((1u << (5u - g)) - 1u);
      const uint32_t v = word < n_words ? bits[word] : 0u;
      any = (v >> (sub << g)) & ((1u << (1u << g)) - 1u);
    }
    out |= (any != 0u ? 1u : 0u) << i;
  }
  coarse[w] = out;
}

template <typename VT>
inline void pack_event_bitmap(hipStream_t stream, const VT *ev, uint32_t n, uint32_t *bits) {
  if (n == 0) return;
  const unsigned groups = div_up(n, kWave);
  const unsigned grid = div_up(groups, 256 / kWave);
  hipLaunchKernelGGL(pack_event_bitmap_kernel<VT>, dim3(grid < 2048 ? grid : 2048), dim3(256), 0, stream, ev, n, bits);
}

__device__ __forceinline__ void atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

}  // namespace bpl
