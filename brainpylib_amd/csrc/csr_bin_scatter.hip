// Transposed CSR matrix times vector: y[c] = sum_j v[row(j)] * data[j] over the nonzeros j of column c.
// Three parts: a dense vector and an output far larger than LDS (hundreds of thousands of columns or more):
// coarse sorting; a dense vector and an output of one or two float64 windows of LDS: a flat walk into the
// windows, no sorting (flat_window_kernel, in the middle of the file); an event vector, where only the listed
// active rows contribute (from 8,192 columns): coarse sorting again (last part).  One random global atomic per
// nonzero retires at about 21 G/s on this device; instead the products are first sorted coarsely:
//
//   bin kernel     persistent producer workgroups take equal shares of the nonzeros (whatever rows they
//                  belong to), form (position in window, product) pairs and append each pair to the bin
//                  of its output window (a power of two of columns, at most 16,384, chosen so that
//                  there are about 64 windows), in a region of scratch memory private to (producer,
//                  window): no global atomics, the position comes from a counter in LDS (32-bit integer
//                  LDS atomics are cheap even when lanes meet).  A pair that does not fit its region (a
//                  share whose columns crowd into few windows) is added to y directly instead.
//   window kernel  workgroup (window, part) adds the pairs of its window from a share of the
//                  producers into a float64 window in LDS (64-bit LDS float adds run at
//                  several lanes per clock) and adds the window to the zeroed y, contiguous.
//
// The arrays are read once, the pairs (6 bytes each: the product, and the position as 16 bits in an array of
// its own) written and read once, in chunks that stay in the cache in front of the memory: HBM bound instead
// of atomic bound.
#include "bins.h"
#include "common.h"
#include "repeated_sum.h"
#include "window_sum.h"

namespace bpl {
namespace {

constexpr int kBinThreads = 1024;
constexpr uint32_t kTileRows = 1024;      // rows staged in LDS at a time by a producer
constexpr uint32_t kMaxWindows = kBinMaxWindows;
constexpr uint32_t kRegionSlack = 128;    // pairs a region holds beyond 5/4 of its even share
constexpr uint32_t kRegionSpacing = kRegionSlack + 8;  // (regions begin and end at multiples of 4 pairs)

// Where producer `p`, whose share is the nonzeros [a0, a1) counted from the first nonzero of the launch, keeps
// the pairs of window b: region_base + b * cap, both multiples of 4 pairs (16-byte loads of the products).
// Both kernels evaluate the same expressions.
__device__ __forceinline__ uint32_t region_cap(uint32_t a0, uint32_t a1, uint32_t n_win) {
  const uint32_t share = (a1 - a0) / n_win;
  return (share + share / 4u + kRegionSlack + 3u) & ~3u;
}
__device__ __forceinline__ uint64_t region_base(uint32_t a0, uint32_t p, uint32_t n_win) {
  return ((static_cast<uint64_t>(a0) + a0 / 4u) & ~3ull) + static_cast<uint64_t>(p) * n_win * kRegionSpacing;
}

// A bin's pairs in memory.  Unpacked: an array of BinPair<F>.  PACKED (windows of at most 2^16 outputs): the
// products in one array of F and the positions within the window in an array of 16-bit words behind it,
// 6 bytes a pair instead of 8 (float) or 10 instead of 16 (double): the pairs are written once and read
// once, which is two thirds of the memory traffic of the transposed product.
typedef float bin_f32x4 __attribute__((ext_vector_type(4)));
typedef double bin_f64x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void load_quad(const float *p, float (&v)[4]) {  // (p: 16-byte aligned)
  const bin_f32x4 t = *reinterpret_cast<const bin_f32x4 *>(p);
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void load_quad(const double *p, double (&v)[4]) {
  const bin_f64x2 a = *reinterpret_cast<const bin_f64x2 *>(p), b = *reinterpret_cast<const bin_f64x2 *>(p + 2);
  v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
}
typedef uint32_t bin_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void load_quad_once(const float *p, float (&v)[4]) {  // (nontemporal)
  const bin_f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const bin_f32x4 *>(p));
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void load_quad_once(const double *p, double (&v)[4]) {
  const bin_f64x2 a = __builtin_nontemporal_load(reinterpret_cast<const bin_f64x2 *>(p));
  const bin_f64x2 b = __builtin_nontemporal_load(reinterpret_cast<const bin_f64x2 *>(p + 2));
  v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
}
// U consecutive columns or weights for a lane, from an address that is a multiple of the element's size only.
// Nontemporal: the arrays pass through once, and lines of pairs that are written a piece per round must stay in
// the L2 until they are whole (120 -> 99 us per 33 million nonzeros; nontemporal STORES of the pairs: 190 us)
typedef uint32_t bin_u32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t bin_u32x2_unaligned __attribute__((ext_vector_type(2), aligned(4)));
typedef float bin_f32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));
typedef double bin_f64x2_unaligned __attribute__((ext_vector_type(2), aligned(8)));
__device__ __forceinline__ void load_consecutive(const uint32_t *p, uint32_t (&c)[4]) {
  const bin_u32x4_unaligned t = __builtin_nontemporal_load(reinterpret_cast<const bin_u32x4_unaligned *>(p));
  c[0] = t.x, c[1] = t.y, c[2] = t.z, c[3] = t.w;
}
__device__ __forceinline__ void load_consecutive(const uint32_t *p, uint32_t (&c)[2]) {
  const bin_u32x2_unaligned t = __builtin_nontemporal_load(reinterpret_cast<const bin_u32x2_unaligned *>(p));
  c[0] = t.x, c[1] = t.y;
}
__device__ __forceinline__ void load_consecutive(const float *p, float (&v)[4]) {
  const bin_f32x4_unaligned t = __builtin_nontemporal_load(reinterpret_cast<const bin_f32x4_unaligned *>(p));
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void load_consecutive(const double *p, double (&v)[2]) {
  const bin_f64x2_unaligned t = __builtin_nontemporal_load(reinterpret_cast<const bin_f64x2_unaligned *>(p));
  v[0] = t.x, v[1] = t.y;
}
__device__ __forceinline__ void load_consecutive(const double *p, double (&v)[4]) {
  const bin_f64x2_unaligned a = __builtin_nontemporal_load(reinterpret_cast<const bin_f64x2_unaligned *>(p));
  const bin_f64x2_unaligned b = __builtin_nontemporal_load(reinterpret_cast<const bin_f64x2_unaligned *>(p + 2));
  v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
}
template <typename F>
struct PackedBins {
  F *val;
  uint16_t *rel;
  __device__ __forceinline__ PackedBins(void *pairs, uint64_t n_pairs)
      : val(static_cast<F *>(pairs)), rel(reinterpret_cast<uint16_t *>(static_cast<F *>(pairs) + n_pairs)) {}
};
template <typename F>
constexpr size_t bin_pair_bytes(bool packed) { return packed ? sizeof(F) + 2 : sizeof(BinPair<F>); }
// The nonzeros [a, b) of producer p: equal shares (multiples of 4) of the launch's nonzeros [lo, hi), whatever
// rows they belong to, so that neither uneven rows nor a matrix of a few long rows leave producers idle.
// lo = chunk_lo; hi = the end of the chunk, or of the matrix for the last chunk (the matrix's nonzero count
// is read on the device: a caller's count that is too small costs speed, not nonzeros).
struct NonzeroShare {
  uint32_t a, b;
};
__device__ __forceinline__ NonzeroShare producer_share(uint32_t nnz, uint32_t chunk_lo, uint32_t chunk_nnz, bool last,
                                                       uint32_t producers, uint32_t p, uint32_t *lo_out) {
  const uint32_t lo = chunk_lo < nnz ? chunk_lo : nnz;
  const uint32_t hi = (last || nnz - lo < chunk_nnz) ? nnz : lo + chunk_nnz;
  const uint32_t per = (static_cast<uint32_t>((static_cast<uint64_t>(hi - lo) + producers - 1u) / producers) + 3u) & ~3u;
  const uint64_t a = static_cast<uint64_t>(lo) + static_cast<uint64_t>(p) * per;
  NonzeroShare s;
  s.a = a < hi ? static_cast<uint32_t>(a) : hi;
  s.b = a + per < hi ? static_cast<uint32_t>(a + per) : hi;
  *lo_out = lo;
  return s;
}

// The last row r in [0, n_row) with indptr[r] <= pos, for pos < indptr[n_row]: the wave searches together,
// 64 probes a round (four rounds for a million rows).
__device__ __forceinline__ uint32_t row_of_nonzero(const uint32_t *__restrict__ indptr, uint32_t n_row, uint32_t pos) {
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  uint32_t lo = 0, hi = n_row;  // indptr[lo] <= pos < indptr[hi]
  while (hi - lo > 1u) {
    const uint32_t span = hi - lo;
    const uint32_t stride = span / kWave + (span % kWave ? 1u : 0u);
    const uint64_t probe = static_cast<uint64_t>(lo) + static_cast<uint64_t>(lane) * stride;
    const bool below = probe < hi && indptr[probe] <= pos;  // (true for lane 0; true lanes form a prefix)
    const uint32_t cnt = static_cast<uint32_t>(__popcll(__ballot(below)));
    lo += (cnt - 1u) * stride;
    hi = (hi - lo > stride) ? lo + stride : hi;
  }
  return lo;
}

constexpr uint32_t kWindowIdShift = 24;  // (positions within a window take kBinMaxShift = 17 bits, window numbers 7)
static_assert(kBinMaxShift <= kWindowIdShift && kBinMaxWindows <= (1u << (32 - kWindowIdShift)), "window id above the position");
constexpr uint32_t kHintShift = 8;                       // one row hint per 256 nonzeros
constexpr uint32_t kSegment = kBinThreads << kHintShift;  // nonzeros covered by one set of hints

template <typename F, bool HETER, bool PACKED>
__global__ __launch_bounds__(kBinThreads) void bin_products_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const F *__restrict__ vec, F *__restrict__ y, uint32_t n_row, uint32_t chunk_lo, uint32_t chunk_nnz, uint32_t last,
    uint32_t n_win, uint32_t shift, void *__restrict__ pairs_raw, uint64_t n_pairs, uint32_t *__restrict__ counts) {
  BinPair<F> *__restrict__ pairs = static_cast<BinPair<F> *>(pairs_raw);
  const PackedBins<F> packed(pairs_raw, n_pairs);
  __shared__ uint32_t s_ptr[kTileRows + 1];
  __shared__ F s_v[kTileRows];
  __shared__ uint32_t s_hint[kBinThreads + 1];  // row (within the tile) of every 256th nonzero of the segment
  __shared__ uint32_t s_cnt[kMaxWindows + 1];   // pairs of the current round, per window (and a spare counter)
  __shared__ uint32_t s_off[kMaxWindows + 1];   // their offsets in the sorted round
  __shared__ uint32_t s_total[kMaxWindows];     // pairs already in this producer's bin, per window
  constexpr int U = (sizeof(F) == 4) ? 4 : 2;
  constexpr uint32_t kRound = U * kBinThreads;
  __shared__ uint32_t s_base[kMaxWindows];
  __shared__ BinPair<F> s_sorted[kRound + 1];  // (and a spare slot; rel: the window's number above the position, from bit kWindowIdShift)
  const uint32_t tid = threadIdx.x;
  const uint32_t p = blockIdx.x;
  if (tid < kMaxWindows) s_cnt[tid] = 0, s_total[tid] = 0;
  if (tid == 0) s_cnt[kMaxWindows] = 0;
  uint32_t chunk_first;
  const NonzeroShare share = producer_share(indptr[n_row], chunk_lo, chunk_nnz, last != 0, gridDim.x, p, &chunk_first);
  const uint32_t a0 = share.a, a1 = share.b;
  const uint32_t cap = region_cap(a0, a1, n_win);
  const uint64_t region_off = region_base(a0 - chunk_first, p, n_win);
  const F w_homo = HETER ? F(0) : data[0];

  // largest k < rows with s_ptr[k] <= j, searched in [lo, hi]
  auto row_of = [&](uint32_t j, uint32_t lo, uint32_t hi) {
    while (lo < hi) {
      const uint32_t mid = (lo + hi + 1u) >> 1;
      if (s_ptr[mid] <= j) lo = mid;
      else hi = mid - 1u;
    }
    return lo;
  };

  // tiles of 1,024 rows from the row that holds nonzero a0 on, until one reaches the end of the share
  for (uint32_t t0 = a0 < a1 ? row_of_nonzero(indptr, n_row, a0) : n_row; t0 < n_row; t0 += kTileRows) {
    const uint32_t rows = (n_row - t0 < kTileRows) ? n_row - t0 : kTileRows;
    __syncthreads();  // the previous tile is done with s_ptr / s_v (and s_cnt is cleared)
    if (tid < rows) s_v[tid] = vec[t0 + tid];
    if (tid <= rows) s_ptr[tid] = indptr[t0 + tid];
    if (tid == 0 && rows == kTileRows) s_ptr[kTileRows] = indptr[t0 + kTileRows];
    __syncthreads();
    const uint32_t tile_end = s_ptr[rows];
    const uint32_t j0 = s_ptr[0] > a0 ? s_ptr[0] : a0, j1 = tile_end < a1 ? tile_end : a1;
    for (uint32_t seg = j0; seg < j1; seg += kSegment) {
      const uint32_t seg_end = (j1 - seg < kSegment) ? j1 : seg + kSegment;
      // A lane takes U consecutive nonzeros of a round: one request for their columns and one for their
      // weights, made a round ahead (before the stores of the round before), one search for the row of the
      // first of them.  The LDS reads and writes of a phase are issued together, without branches around them
      // (a nonzero beyond the segment counts in a spare counter and is sorted into a spare slot): between two
      // barriers a wave waits for LDS two or three times, not once per nonzero.
      uint32_t col[U];
      F dat[U];
      auto load_round = [&](uint32_t base) {
        const uint32_t j = base + U * tid;
        if (j + U <= seg_end) {
          load_consecutive(indices + j, col);
          if (HETER) load_consecutive(data + j, dat);
        } else {
#pragma unroll
          for (int t = 0; t < U; ++t) {
            const uint32_t jc = j + t < seg_end ? j + t : seg_end - 1u;
            col[t] = indices[jc];
            if (HETER) dat[t] = data[jc];
          }
        }
      };
      load_round(seg);
      // hints: the row of nonzero seg + 256 q, for every q up to the end of the segment
      __syncthreads();  // the previous segment is done with s_hint
      {
        const uint32_t j = seg + (tid << kHintShift);
        s_hint[tid] = (j < seg_end) ? row_of(j, 0u, rows - 1u) : rows - 1u;
        if (tid == 0) s_hint[kBinThreads] = rows - 1u;
      }
      __syncthreads();
      // Rounds of kRound nonzeros.  The round's pairs are first sorted by window in LDS (rank within
      // the window from an LDS counter, window offsets from a scan of the counters), then written
      // out in that order: pairs of one window go to consecutive addresses of its bin, so the
      // stores of neighbouring lanes merge instead of arriving as single 8-byte requests.
      for (uint32_t base = seg; base < seg_end; base += kRound) {
        const uint32_t j = base + U * tid;
        uint32_t rank[U], win[U], rel[U], krow[U];
        F val[U], v[U];
        {
          const uint32_t jf = j < seg_end ? j : seg_end - 1u;
          const uint32_t q = (jf - seg) >> kHintShift;
          uint32_t kk = row_of(jf, s_hint[q], s_hint[q + 1]);
          uint32_t e = s_ptr[kk + 1u];
#pragma unroll
          for (int t = 0; t < U; ++t) {
            const uint32_t jt = j + t < seg_end ? j + t : seg_end - 1u;
            while (e <= jt) e = s_ptr[++kk + 1u];  // (ends: jt < seg_end <= s_ptr[rows])
            krow[t] = kk;
          }
        }
#pragma unroll
        for (int t = 0; t < U; ++t) v[t] = s_v[krow[t]];
#pragma unroll
        for (int t = 0; t < U; ++t) {
          // v * values[j] (heter) or values * v (homo), as the reference's CPU loop multiplies
          val[t] = HETER ? static_cast<F>(v[t] * dat[t]) : static_cast<F>(w_homo * v[t]);
          win[t] = j + t < seg_end ? col[t] >> shift : kMaxWindows;  // (kMaxWindows: no pair)
          rel[t] = col[t] & ((1u << shift) - 1u);
        }
        // (Long rows with their columns in order: all of a wave's nonzeros fall into one window, and as many
        // atomics on one counter would take their turns.  One lane then reserves the ranks of the whole wave.)
        bool one_window = true;
        const uint32_t w_first = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(win[0])));
#pragma unroll
        for (int t = 0; t < U; ++t) one_window = one_window && win[t] == w_first;
        if (__all(one_window)) {
          uint32_t first_rank = 0;
          if (tid % kWave == 0) first_rank = atomicAdd(&s_cnt[w_first], static_cast<uint32_t>(U * kWave));
          first_rank = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(first_rank)));
#pragma unroll
          for (int t = 0; t < U; ++t) rank[t] = first_rank + U * (tid % kWave) + t;
        } else {
#pragma unroll
          for (int t = 0; t < U; ++t) rank[t] = atomicAdd(&s_cnt[win[t]], 1u);
        }
        __syncthreads();
        if (tid < kWave) {  // offsets of the windows within the round: two counters per lane
          const uint32_t c0 = s_cnt[2 * tid], c1 = s_cnt[2 * tid + 1];
          const uint32_t incl = wave_inclusive_scan_u32(c0 + c1);
          const uint32_t o0 = incl - (c0 + c1), o1 = incl - c1;
          s_off[2 * tid] = o0;
          s_off[2 * tid + 1] = o1;
          if (tid == kWave - 1) s_off[kMaxWindows] = incl;
          // slot in the bin of the pair at position i of the sorted round: s_base[window] + i (modulo 2^32)
          const uint32_t t0w = s_total[2 * tid], t1w = s_total[2 * tid + 1];
          s_base[2 * tid] = t0w - o0;
          s_base[2 * tid + 1] = t1w - o1;
          s_total[2 * tid] = t0w + c0;
          s_total[2 * tid + 1] = t1w + c1;
          s_cnt[2 * tid] = 0;
          s_cnt[2 * tid + 1] = 0;
        }
        __syncthreads();
        uint32_t pos[U];
#pragma unroll
        for (int t = 0; t < U; ++t) pos[t] = s_off[win[t]];
#pragma unroll
        for (int t = 0; t < U; ++t) {
          BinPair<F> e;
          e.rel = rel[t] | (win[t] << kWindowIdShift);
          e.val = val[t];
          s_sorted[win[t] != kMaxWindows ? pos[t] + rank[t] : kRound] = e;
        }
        __syncthreads();
        // (No barrier behind the stores: the next round's counting follows at once; what the stores read is
        // written again only behind the next round's barriers.)
        if (base + kRound < seg_end) load_round(base + kRound);
        const uint32_t round_total = s_off[kMaxWindows];
        BinPair<F> out[U];
        uint32_t slot0[U];
#pragma unroll
        for (int u = 0; u < U; ++u) out[u] = s_sorted[tid + u * kBinThreads];  // (beyond the round's total: stale, unused)
#pragma unroll
        for (int u = 0; u < U; ++u) slot0[u] = s_base[(out[u].rel >> kWindowIdShift) % kMaxWindows];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t i = tid + u * kBinThreads;
          if (i < round_total) {
            const uint32_t w = out[u].rel >> kWindowIdShift;
            const uint32_t r = out[u].rel & ((1u << kWindowIdShift) - 1u);
            const uint32_t slot = slot0[u] + i;
            const uint64_t at = region_off + static_cast<uint64_t>(w) * cap + slot;
            if (slot < cap && at < n_pairs) {
              if (PACKED) {
                packed.val[at] = out[u].val, packed.rel[at] = static_cast<uint16_t>(r);
              } else {
                BinPair<F> e;
                e.rel = r, e.val = out[u].val;
                pairs[at] = e;
              }
            } else {
              atomic_add(y + ((w << shift) | r), out[u].val);
            }
          }
        }
      }
    }
    if (tile_end >= a1) break;
  }
  if (tid < n_win) {
    const uint32_t c = s_total[tid];
    counts[static_cast<size_t>(tid) * gridDim.x + p] = c < cap ? c : cap;
  }
}

// ---- one output window ------------------------------------------------------------------------
// Transposed product whose output fits ONE float64 window in LDS (up to 16,384 columns): no sorting.
// Every workgroup takes a contiguous range of the NONZEROS (whatever rows they belong to, so that
// uneven rows and hub rows cost nothing), walks it like the producer above (a lane takes U consecutive
// nonzeros with one 16-byte request each for columns and weights, one search for the row of the first)
// and adds the products to its window with float64 LDS atomics; there is no barrier inside a tile of
// 1,024 rows.  The windows go to scratch memory as float64 and a second kernel adds them in a fixed
// order and rounds once.  (A wave per row, as the window kernel of the event operators walks, leaves
// most lanes idle on short rows: 1,000,000 x 16,000 with 100 per row 616 us, 4,000,000 x 8,000 with
// 20 per row 1,510 us.)
template <typename F, bool HETER>
__global__ __launch_bounds__(kBinThreads) void flat_window_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const F *__restrict__ vec, uint32_t n_row, uint32_t n_col, uint32_t slices, double *__restrict__ partial) {
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  double *window = reinterpret_cast<double *>(smem_raw);
  // workgroup (share, slice): the share's nonzeros whose columns lie in slice `slice` of the output (one slice
  // unless the output is wider than a window: every slice's workgroups then read the share again)
  const uint32_t shares = gridDim.x / slices, share = blockIdx.x / slices, slice = blockIdx.x % slices;
  const uint32_t c_lo = slice * kFlatWindowMaxCols;
  const uint32_t width = n_col - c_lo < kFlatWindowMaxCols ? n_col - c_lo : kFlatWindowMaxCols;
  __shared__ uint32_t s_ptr[kTileRows + 1];
  __shared__ F s_v[kTileRows];
  __shared__ uint32_t s_hint[kBinThreads + 1];  // row (within the tile) of every 256th nonzero of the segment
  constexpr int U = (sizeof(F) == 4) ? 4 : 2;
  constexpr uint32_t kRound = U * kBinThreads;
  const uint32_t tid = threadIdx.x;
  for (uint32_t i = tid; i < width; i += kBinThreads) window[i] = 0.0;
  const uint32_t nnz = indptr[n_row];
  // the share's nonzeros [a, b): equal shares, multiples of 4
  const uint32_t per = (static_cast<uint32_t>((static_cast<uint64_t>(nnz) + shares - 1u) / shares) + 3u) & ~3u;
  const uint64_t a64 = static_cast<uint64_t>(share) * per;
  const uint32_t a = a64 < nnz ? static_cast<uint32_t>(a64) : nnz;
  const uint32_t b = a64 + per < nnz ? static_cast<uint32_t>(a64 + per) : nnz;
  const F w_homo = HETER ? F(0) : data[0];

  // largest k in [lo, hi] with s_ptr[k] <= j
  auto row_of = [&](uint32_t j, uint32_t lo, uint32_t hi) {
    while (lo < hi) {
      const uint32_t mid = (lo + hi + 1u) >> 1;
      if (s_ptr[mid] <= j) lo = mid;
      else hi = mid - 1u;
    }
    return lo;
  };

  if (a < b) {
    uint32_t t0 = row_of_nonzero(indptr, n_row, a);  // the row that holds nonzero a
    for (;;) {
      const uint32_t rows = (n_row - t0 < kTileRows) ? n_row - t0 : kTileRows;
      __syncthreads();  // the previous tile is done with s_ptr / s_v (and the window is cleared)
      if (tid < rows) s_v[tid] = vec[t0 + tid];
      if (tid <= rows) s_ptr[tid] = indptr[t0 + tid];
      if (tid == 0 && rows == kTileRows) s_ptr[kTileRows] = indptr[t0 + kTileRows];
      __syncthreads();
      const uint32_t tile_end = s_ptr[rows];
      const uint32_t j0 = s_ptr[0] > a ? s_ptr[0] : a, j1 = tile_end < b ? tile_end : b;
      for (uint32_t seg = j0; seg < j1; seg += kSegment) {
        const uint32_t seg_end = (j1 - seg < kSegment) ? j1 : seg + kSegment;
        __syncthreads();  // the previous segment is done with s_hint
        {
          const uint32_t j = seg + (tid << kHintShift);
          s_hint[tid] = (j < seg_end) ? row_of(j, 0u, rows - 1u) : rows - 1u;
          if (tid == 0) s_hint[kBinThreads] = rows - 1u;
        }
        __syncthreads();
        for (uint32_t base = seg; base < seg_end; base += kRound) {
          const uint32_t j = base + U * tid;
          if (j >= seg_end) continue;
          uint32_t col[U];
          F dat[U];
          if (j + U <= seg_end) {
            load_consecutive(indices + j, col);
            if (HETER) load_consecutive(data + j, dat);
          } else {
#pragma unroll
            for (int t = 0; t < U; ++t) {
              const uint32_t jc = j + t < seg_end ? j + t : seg_end - 1u;
              col[t] = indices[jc];
              if (HETER) dat[t] = data[jc];
            }
          }
          const uint32_t q = (j - seg) >> kHintShift;
          uint32_t kk = row_of(j, s_hint[q], s_hint[q + 1]);
          uint32_t e = s_ptr[kk + 1u];
          uint32_t krow[U];
#pragma unroll
          for (int t = 0; t < U; ++t) {
            const uint32_t jt = j + t < seg_end ? j + t : seg_end - 1u;
            while (e <= jt) e = s_ptr[++kk + 1u];  // (ends: jt < seg_end <= s_ptr[rows])
            krow[t] = kk;
          }
          F v[U];
#pragma unroll
          for (int t = 0; t < U; ++t) v[t] = s_v[krow[t]];
#pragma unroll
          for (int t = 0; t < U; ++t) {
            // v * values[j] (heter) or values * v (homo), as the reference's CPU loop multiplies
            const F prod = HETER ? static_cast<F>(v[t] * dat[t]) : static_cast<F>(w_homo * v[t]);
            if (j + t < seg_end && col[t] - c_lo < width) atomicAdd(&window[col[t] - c_lo], static_cast<double>(prod));  // (wraps below c_lo)
          }
        }
      }
      if (tile_end >= b || t0 + rows >= n_row) break;
      t0 += rows;
    }
  }
  __syncthreads();
  double *mine = partial + static_cast<size_t>(share) * n_col + c_lo;
  for (uint32_t i = tid; i < width; i += kBinThreads) mine[i] = window[i];
}

// y[c] = the sum of the workgroups' windows in a fixed order, in float64, rounded once.
template <typename F>
__global__ __launch_bounds__(kSumCols * kSumSlices) void sum_windows_kernel(const double *__restrict__ partial,
                                                                            F *__restrict__ y, uint32_t n_col,
                                                                            uint32_t groups) {
  bool mine;
  const double total = sum_windows_of_column<double, double>(partial, n_col, groups, &mine);
  if (mine) y[blockIdx.x * kSumCols + threadIdx.x % kSumCols] = static_cast<F>(total);
}

// grid = n_win * slices * parts; workgroup (b, q, s) adds window b's pairs of producers
// [s * P / parts, ...) that fall into slice q of the window (slices = 2^(shift - lds_shift): a window
// wider than the 2^lds_shift accumulators in LDS is added slice by slice, every slice reading the pairs).
// Bin of (producer p, window b): derived from the producers' shares of the nonzeros as in bin_products_kernel,
// or, with indptr == nullptr, the uniform layout pairs + (p * n_win + b) * uniform_cap.
// ONCE: the pairs are read with nontemporal loads (bins of a jitconn column walk: gigabytes that passed
// through memory; 1e8 pairs: 524 -> 484 us with the walk).  The CSR product's chunks come back from the
// cache in front of the memory, where the hint costs (454 -> 510 us).
template <typename F, bool PACKED, bool ONCE>
__global__ __launch_bounds__(kBinThreads) void add_bins_kernel(const uint32_t *__restrict__ indptr,
                                                               F *__restrict__ y, uint32_t n_row, uint32_t n_col,
                                                               uint32_t chunk_lo, uint32_t chunk_nnz, uint32_t last,
                                                               uint32_t n_win, uint32_t shift,
                                                               uint32_t lds_shift, uint32_t parts,
                                                               uint32_t producers,
                                                               const void *__restrict__ pairs_raw,
                                                               uint64_t n_pairs,
                                                               const uint32_t *__restrict__ counts,
                                                               uint32_t uniform_cap, uint32_t *__restrict__ reset) {
  const BinPair<F> *__restrict__ pairs = static_cast<const BinPair<F> *>(pairs_raw);
  const PackedBins<F> packed(const_cast<void *>(pairs_raw), n_pairs);
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  // (a counter of the producer's, left at zero for the next call)
  if (reset != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *reset = 0u;
  double *window = reinterpret_cast<double *>(smem_raw);
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  constexpr uint32_t kWaves = kBinThreads / kWave;
  const uint32_t slices = 1u << (shift - lds_shift);
  const uint32_t b = blockIdx.x / (parts * slices), q = (blockIdx.x / parts) % slices, s = blockIdx.x % parts;
  const uint32_t r0 = q << lds_shift;  // first column of the slice within the window
  const uint32_t c0 = (b << shift) + r0;
  if (c0 >= n_col) return;
  const uint32_t width = (n_col - c0 < (1u << lds_shift)) ? n_col - c0 : (1u << lds_shift);
  for (uint32_t i = tid; i < width; i += kBinThreads) window[i] = 0.0;
  __syncthreads();
  const uint32_t nnz_all = indptr != nullptr ? indptr[n_row] : 0u;
  const uint32_t p_lo = static_cast<uint32_t>(static_cast<uint64_t>(s) * producers / parts);
  const uint32_t p_hi = static_cast<uint32_t>(static_cast<uint64_t>(s + 1) * producers / parts);
  // A wave takes the bins of the producers p_lo + wave, + kWaves, ... one after the other, in steps of
  // 8 pairs per lane; where the bins are and how many pairs they hold is fetched for 64 bins at once
  // (one per lane).  The steps of consecutive bins form ONE sequence, and a step's pairs are requested
  // before the step before it is added: two steps (16 pairs per lane) are in flight, and a wave that
  // walks many small bins (a jitconn column walk leaves a few hundred pairs in each) does not pay a
  // round trip per bin.
  constexpr int kAddU = 8;
  uint32_t g0 = p_lo + wave;  // producer of lane 0's bin in the current block of 64 bins
  uint32_t j = kWave;         // bin of the block the sequence is in (kWave: fetch a block first)
  bool first_block = true;
  uint64_t my_off = 0;
  uint32_t my_n = 0;
  const BinPair<F> *bin = nullptr;
  uint64_t bin_off = 0;  // (in pairs)
  uint32_t n = 0, i0 = 0, i_next = 0;
  auto next_step = [&]() -> bool {  // moves (bin, n, i0) on; false at the end of the wave's share (wave uniform)
    for (;;) {
      if (i_next < n) {
        i0 = i_next;
        i_next += kAddU * kWave;
        return true;
      }
      ++j;
      if (j >= static_cast<uint32_t>(kWave) || static_cast<uint64_t>(g0) + static_cast<uint64_t>(j) * kWaves >= p_hi) {
        if (!first_block) {
          if (static_cast<uint64_t>(g0) + static_cast<uint64_t>(kWaves) * kWave >= p_hi) return false;
          g0 += kWaves * kWave;
        } else if (g0 >= p_hi) {
          return false;
        }
        first_block = false;
        my_off = 0;
        my_n = 0;
        const uint64_t p64 = static_cast<uint64_t>(g0) + static_cast<uint64_t>(lane) * kWaves;
        if (p64 < p_hi) {
          const uint32_t p = static_cast<uint32_t>(p64);
          if (indptr != nullptr) {
            uint32_t chunk_first;
            const NonzeroShare share = producer_share(nnz_all, chunk_lo, chunk_nnz, last != 0, producers, p, &chunk_first);
            my_off = region_base(share.a - chunk_first, p, n_win) + static_cast<uint64_t>(b) * region_cap(share.a, share.b, n_win);
          } else {
            my_off = (static_cast<uint64_t>(p) * n_win + b) * uniform_cap;
          }
          my_n = counts[static_cast<size_t>(b) * producers + p];
          if (indptr == nullptr && my_n > uniform_cap) my_n = uniform_cap;  // the producer counts what it could not store too
          if (my_off >= n_pairs) my_n = 0;  // (only if the caller's nonzero count was too small)
          else if (my_n > n_pairs - my_off) my_n = static_cast<uint32_t>(n_pairs - my_off);
        }
        j = 0;
      }
      n = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(my_n), j));
      const uint32_t off_lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(my_off), j));
      const uint32_t off_hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(my_off >> 32), j));
      bin_off = (static_cast<uint64_t>(off_hi) << 32) | off_lo;
      bin = pairs + bin_off;
      i_next = 0;
    }
  };
  // Every step issues the same loads whatever it holds (a lane beyond the bin's count reads the bin's first
  // pairs again and leaves them out by their number; behind the last step come empty ones): the compiler can
  // then count the loads in flight and wait for one step's while the next ones' are on their way.  With loads
  // inside branches it waits for all of them before it issues more.
  struct PairStep {
    BinPair<F> p[kAddU];
    uint32_t left;  // pairs from the step's first one to the end of the bin
  };
  auto load_pairs = [&](PairStep &e) {
    e.left = i0 < n ? n - i0 : 0u;
#pragma unroll
    for (int u = 0; u < kAddU; ++u) {
      const uint32_t i = i0 + u * kWave + lane;
      e.p[u] = bin[i < n ? i : 0u];
    }
  };
  auto add_pairs = [&](const PairStep &e) {
#pragma unroll
    for (int u = 0; u < kAddU; ++u)
      if (u * kWave + lane < e.left && e.p[u].rel - r0 < width)
        atomicAdd(&window[e.p[u].rel - r0], static_cast<double>(e.p[u].val));  // (wraps below r0)
  };
  // Packed bins: a lane takes two quads of a step, each 16 or 32 bytes of products and 8 bytes of positions
  // (bins begin at multiples of 4 pairs and their regions end at one: a bin's last quad is read whole and
  // its elements beyond the count are left out by their number).
  struct PackedStep {
    F v[2][4];
    uint32_t r[2][2];  // four 16-bit positions
    uint32_t valid[2];
  };
  auto load_packed = [&](PackedStep &e) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t i = i0 + 4u * (static_cast<uint32_t>(u) * kWave + lane);
      e.valid[u] = i < n ? n - i : 0u;
      const uint64_t at = bin_off + (i < n ? i : 0u);
      if constexpr (ONCE) {
        const bin_u32x2 r = __builtin_nontemporal_load(reinterpret_cast<const bin_u32x2 *>(packed.rel + at));
        e.r[u][0] = r.x, e.r[u][1] = r.y;
        load_quad_once(packed.val + at, e.v[u]);
      } else {
        const uint2 r = *reinterpret_cast<const uint2 *>(packed.rel + at);
        e.r[u][0] = r.x, e.r[u][1] = r.y;
        load_quad(packed.val + at, e.v[u]);
      }
    }
  };
  auto add_packed = [&](const PackedStep &e) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t rel = (e.r[u][t / 2] >> (16 * (t % 2))) & 0xffffu;
        if (static_cast<uint32_t>(t) < e.valid[u] && rel - r0 < width)
          atomicAdd(&window[rel - r0], static_cast<double>(e.v[u][t]));  // (wraps below r0)
      }
    }
  };
  // D steps are under way at a time; step k is added when step k + D - 1 has been requested.
  auto run = [&](auto &e, auto load, auto add) {
    constexpr int D = static_cast<int>(sizeof(e) / sizeof(e[0]));
    bool live = next_step();
    if (!live) return;
    uint64_t last_off = bin_off;  // a bin that holds pairs: what an empty step reads
    auto advance = [&]() {
      live = live && next_step();
      if (live) last_off = bin_off;
      else n = 0, bin_off = last_off, bin = pairs + last_off;
    };
    bool has[D];
    load(e[0]);
    has[0] = true;
#pragma unroll
    for (int d = 1; d < D - 1; ++d) {
      advance();
      load(e[d]);
      has[d] = live;
    }
    for (;;) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int nx = (d + D - 1) % D;
        advance();
        load(e[nx]);
        has[nx] = live;
        add(e[d]);
        if (!has[(d + 1) % D]) return;
      }
    }
  };
  if (PACKED) {
    PackedStep e[4];
    run(e, load_packed, add_packed);
  } else {
    PairStep e[2];
    run(e, load_pairs, add_pairs);
  }
  __syncthreads();
  for (uint32_t i = tid; i < width; i += kBinThreads) {
    const F v = static_cast<F>(window[i]);
    if (v != F(0)) atomic_add(y + c0 + i, v);
  }
}

// Homogeneous weight, event input: the reference adds the weight once per synapse, in place, in the
// precision of the output, so an output is a function of its synapse count alone (repeated_sum.h).
// Pairs that do not fit their run are counted in the output element's own storage (zeroed before:
// float, the 32 bits as an integer; double, the count as a number), and the workgroup that owns
// the element adds the pairs it counted in LDS and stores the sum.
__device__ __forceinline__ void add_synapse_count(float *y, uint32_t n) { atomicAdd(reinterpret_cast<uint32_t *>(y), n); }
__device__ __forceinline__ void add_synapse_count(double *y, uint32_t n) { atomic_add(y, static_cast<double>(n)); }
__device__ __forceinline__ uint64_t synapse_count(float v) { return __float_as_uint(v); }
__device__ __forceinline__ uint64_t synapse_count(double v) { return static_cast<uint64_t>(v); }

// ---- event input -------------------------------------------------------------------------------
// Only the active rows contribute, how many is known on the device alone (a list made by the
// caller: (first nonzero, length) per active row, their number in active_count[0]), and the
// descriptor of the event operators does not carry the nonzero count.  So the bins are not private
// to a producer here: window b owns 8 runs of `cap` pairs each, shared by the producers p with the
// same p % 8, and a producer reserves room for the pairs a round holds for a window with one
// global atomic on the run's fill counter (at most one per window and round of 4,096 nonzeros;
// the event operators move far fewer pairs than the dense product, for which that many
// same-address atomics would cost more than private regions).  Whatever the distribution of the
// activity over rows and of the columns over windows, a run only overflows (into direct atomics
// on y) when it receives more than `cap` pairs.
constexpr uint32_t kPairsPerProducer = 4096;  // a producer takes part per that many active nonzeros (estimated): one round
constexpr uint32_t kSubRuns = 8;              // a window's run is split: producer p appends to sub-run p % 8, so that
                                              // the atomics on one counter (about 15 ns each) stay few
constexpr uint32_t kFillStride = 32;          // words between fill counters: one 128-byte line each
static_assert(kBinEventFillBytes == kMaxWindows * kSubRuns * kFillStride * sizeof(uint32_t),
              "one fill counter per window and sub-run");
constexpr uint32_t kPairsPerPart = 8192;      // a consumer workgroup takes part per that many pairs of its window
// Little activity (the usual state of a spiking network): up to this many active nonzeros
// (estimated) skip the runs, because the chain list -> sort -> reserve -> store -> add costs more
// than their atomics.  The producer only leaves the number of active rows in a spare word of the
// fill area (zeroed with it before every call) and the consumer's waves add the rows to y directly.
constexpr uint32_t kDirectPairs = 131072;
constexpr uint32_t kDirectWord = 1;           // (fill counters sit at multiples of kFillStride)

// (At most 80 scalar registers: measured on this device, a 1,024-thread workgroup whose waves hold
// 81..96 of them is alone on its CU, as it would be with more than 64 vector registers; the
// float producer crossed that line by one register and took 37 instead of 27 us.)
template <typename F, bool HETER, typename I>
__global__ __launch_bounds__(kBinThreads) __attribute__((amdgpu_num_sgpr(80))) void bin_active_rows_kernel(
    const F *__restrict__ data, const I *__restrict__ indices, const I *__restrict__ indptr,
    uint32_t n_row, const uint32_t *__restrict__ active_count, const uint2 *__restrict__ active_list,
    uint32_t list_cap, const uint32_t *__restrict__ active_colbase, F *__restrict__ y, uint32_t shift, uint32_t cap,
    BinPair<F> *__restrict__ pairs, uint32_t *__restrict__ fill) {
  __shared__ uint32_t s_ptr[kTileRows + 1];     // nonzeros of the tile's rows before row k
  __shared__ uint32_t s_start[kTileRows];       // first nonzero of row k in the matrix
  __shared__ uint32_t s_colbase[kTileRows];     // added to row k's columns (batched calls: batch entry * n_col)
  __shared__ uint32_t s_hint[kBinThreads + 1];
  __shared__ uint32_t s_cnt[kMaxWindows];
  __shared__ uint32_t s_off[kMaxWindows + 1];
  __shared__ uint32_t s_base[kMaxWindows];      // where the round's pairs of a window go in its run
  __shared__ uint32_t s_wave[kBinThreads / kWave];
  constexpr int U = (sizeof(F) == 4) ? 4 : 2;
  constexpr uint32_t kRound = U * kBinThreads;
  __shared__ BinPair<F> s_sorted[kRound];
  __shared__ uint8_t s_window[kRound];
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const uint32_t total = active_count[0] < list_cap ? active_count[0] : list_cap;  // (never beyond the list)
  const uint32_t nnz = static_cast<uint32_t>(indptr[n_row]);  // (64-bit offsets: listed only below 2^32 nonzeros)
  // with little activity a few producers finish sooner than a chip full of them
  const uint64_t want = (static_cast<uint64_t>(total) * (nnz / n_row + 1u) + kPairsPerProducer - 1u) / kPairsPerProducer;
  const uint32_t producers = want < 1u ? 1u : want > gridDim.x ? gridDim.x : static_cast<uint32_t>(want);
  if (static_cast<uint64_t>(total) * (nnz / n_row + 1u) <= kDirectPairs) {
    if (blockIdx.x == 0 && tid == 0) fill[kDirectWord] = total;
    return;
  }
  const uint32_t p = blockIdx.x;
  if (p >= producers) return;
  const uint32_t sub = p % kSubRuns;
  // Producer p takes an equal share of the listed rows; where there are fewer rows than producers (a few
  // long rows are active), `parts` producers take a row, each an equal part of its nonzeros.
  uint32_t lo, hi, part = 0, parts = 1;
  if (total < producers) {
    parts = producers / total;
    lo = p / parts, hi = lo + 1u, part = p % parts;
    if (lo >= total) return;
  } else {
    lo = static_cast<uint32_t>(static_cast<uint64_t>(p) * total / producers);
    hi = static_cast<uint32_t>(static_cast<uint64_t>(p + 1) * total / producers);
  }
  if (tid < kMaxWindows) s_cnt[tid] = 0;
  const F w_homo = HETER ? F(0) : data[0];
  // homogeneous weight: a run holds the pairs' columns only, `cap` of them
  uint32_t *run_columns = reinterpret_cast<uint32_t *>(pairs);

  auto row_of = [&](uint32_t j, uint32_t a, uint32_t b) {  // largest k in [a, b] with s_ptr[k] <= j
    while (a < b) {
      const uint32_t mid = (a + b + 1u) >> 1;
      if (s_ptr[mid] <= j) a = mid;
      else b = mid - 1u;
    }
    return a;
  };

  for (uint32_t t0 = lo; t0 < hi; t0 += kTileRows) {
    const uint32_t rows = (hi - t0 < kTileRows) ? hi - t0 : kTileRows;
    __syncthreads();  // the previous tile is done with s_ptr / s_start (and s_cnt is cleared)
    uint2 e = make_uint2(0u, 0u);
    if (tid < rows) e = active_list[t0 + tid];
    if (parts > 1u) {  // (one row: this producer's part of it, which may be empty)
      const uint32_t a = static_cast<uint32_t>(static_cast<uint64_t>(e.y) * part / parts);
      const uint32_t b = static_cast<uint32_t>(static_cast<uint64_t>(e.y) * (part + 1u) / parts);
      e.x += a, e.y = b - a;
    }
    const uint32_t incl = wave_inclusive_scan_u32(e.y);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave[w];
    if (tid < rows) {
      s_ptr[tid] = before + incl - e.y, s_start[tid] = e.x;
      s_colbase[tid] = active_colbase ? active_colbase[t0 + tid] : 0u;
    }
    if (tid == rows - 1u) s_ptr[rows] = before + incl;
    __syncthreads();
    const uint32_t j1 = s_ptr[rows];  // the tile's nonzeros, numbered from 0 (listed rows are never empty)
    for (uint32_t seg = 0; seg < j1; seg += kSegment) {
      const uint32_t seg_end = (j1 - seg < kSegment) ? j1 : seg + kSegment;
      __syncthreads();  // the previous segment is done with s_hint
      {
        const uint32_t j = seg + (tid << kHintShift);
        s_hint[tid] = (j < seg_end) ? row_of(j, 0u, rows - 1u) : rows - 1u;
        if (tid == 0) s_hint[kBinThreads] = rows - 1u;
      }
      __syncthreads();
      // One round's column indices and weights are requested a round ahead, so that their latency
      // overlaps the sort, the reservation and the stores of the round before.
      auto fetch = [&](uint32_t jb, uint32_t (&col)[U], F (&val)[U]) {
        // first where every nonzero of the lane lies (LDS only), then all the loads together, without a
        // branch around them (beyond the segment: its last nonzero again)
        uint32_t at[U], cb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t j = jb + u * kBinThreads;
          const uint32_t jc = j < seg_end ? j : seg_end - 1u;
          const uint32_t q = (jc - seg) >> kHintShift;
          const uint32_t k = row_of(jc, s_hint[q], s_hint[q + 1]);
          at[u] = s_start[k] + (jc - s_ptr[k]);
          cb[u] = s_colbase[k];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          col[u] = static_cast<uint32_t>(indices[at[u]]);
          val[u] = HETER ? data[at[u]] : w_homo;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t j = jb + u * kBinThreads;
          col[u] = j < seg_end ? col[u] + cb[u] : 0xffffffffu;  // (0xffffffff: no pair)
        }
      };
      uint32_t col[U];
      F val[U];
      fetch(seg + tid, col, val);
      for (uint32_t jb = seg + tid; jb - tid < seg_end; jb += kRound) {
        uint32_t ncol[U];
        F nval[U];
#pragma unroll
        for (int u = 0; u < U; ++u) ncol[u] = 0xffffffffu, nval[u] = F(0);
        if (jb - tid + kRound < seg_end) fetch(jb + kRound, ncol, nval);
        uint32_t rank[U], win[U], rel[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          rank[u] = 0;
          win[u] = 0xffffffffu;
          rel[u] = 0;
          if (col[u] != 0xffffffffu) {
            win[u] = col[u] >> shift;
            rel[u] = col[u] & ((1u << shift) - 1u);
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (win[u] != 0xffffffffu) rank[u] = atomicAdd(&s_cnt[win[u]], 1u);
        __syncthreads();
        if (tid < kWave) {  // two windows per lane: offsets within the round, room in the windows' runs
          const uint32_t c0 = s_cnt[2 * tid], c1 = s_cnt[2 * tid + 1];
          const uint32_t sum = wave_inclusive_scan_u32(c0 + c1);
          s_off[2 * tid] = sum - (c0 + c1);
          s_off[2 * tid + 1] = sum - c1;
          if (tid == kWave - 1) s_off[kMaxWindows] = sum;
          // (both reservations under way together; a window without pairs adds nothing to its counter)
          const uint32_t b0 = atomicAdd(&fill[(2 * tid * kSubRuns + sub) * kFillStride], c0);
          const uint32_t b1 = atomicAdd(&fill[((2 * tid + 1) * kSubRuns + sub) * kFillStride], c1);
          s_base[2 * tid] = b0;
          s_base[2 * tid + 1] = b1;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (win[u] != 0xffffffffu) {
            const uint32_t pos = s_off[win[u]] + rank[u];
            BinPair<F> o;
            o.rel = rel[u];
            o.val = val[u];
            s_sorted[pos] = o;
            s_window[pos] = static_cast<uint8_t>(win[u]);
          }
        }
        __syncthreads();
        const uint32_t round_total = s_off[kMaxWindows];
        for (uint32_t i = tid; i < round_total; i += kBinThreads) {
          const uint32_t w = s_window[i];
          const BinPair<F> o = s_sorted[i];
          const uint32_t slot = s_base[w] + (i - s_off[w]);
          if (slot < cap) {
            if (HETER) pairs[static_cast<uint64_t>(w * kSubRuns + sub) * cap + slot] = o;
            else run_columns[static_cast<uint64_t>(w * kSubRuns + sub) * cap + slot] = o.rel;
          } else if (HETER) atomic_add(y + ((w << shift) | o.rel), o.val);
          else add_synapse_count(y + ((w << shift) | o.rel), 1u);  // (the consumer turns counts into sums)
        }
        __syncthreads();
        if (tid < kMaxWindows) s_cnt[tid] = 0;
        __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) col[u] = ncol[u], val[u] = nval[u];
      }
    }
  }
}

// ---- event input, one output window ----------------------------------------------------------------
// Outputs of at most 8,192 columns and a list of active rows: no sorting, the producers' flat walk over the
// listed rows' nonzeros adds straight into a window in LDS (float64 for weights; 32-bit synapse counts for a
// homogeneous weight, whose sum is formed from the count as everywhere), two workgroups per CU, no barrier
// inside a tile of 1,024 listed rows.  The windows of the workgroups that took part go to scratch memory
// and a second kernel adds them in a fixed order.  (The window kernel of csr_ops.hip hands whole rows to
// waves, one after the other: 1,000,000 rows of 100 into 4,000 columns at 5 % events 76 us, this one 38.)
constexpr uint32_t kWindowEventMaxCols = 8192;

// Workgroups that take part.  P of them walk pairs / P active nonzeros each (estimated from the mean row length) and
// then each writes its window of `window_bytes` for the kernel that adds the windows to read: the two costs are
// equal where a workgroup takes sqrt(pairs * window_bytes / c) nonzeros, c = the cost of a byte of window over the
// cost of a nonzero: measured 300 with one weight, 600 with weights per nonzero (a float64 atomic per nonzero).
// (4,096 per workgroup whatever the window: 50,000 x 50,000 with 200 per row, one weight, at 1 / 5 % events 20 / 31 us
// instead of 17 / 23; 32,000 x 8,192 with 1,000 per row at 5 % 24 instead of 19.5, with weights 21 instead of 19.)
__device__ __forceinline__ uint32_t window_event_producers(uint32_t total, uint32_t nnz, uint32_t n_row, uint32_t launched,
                                                           uint32_t window_bytes, bool heter) {
  const uint64_t pairs = static_cast<uint64_t>(total) * (nnz / n_row + 1u);
  float each = __builtin_sqrtf(static_cast<float>(pairs) * static_cast<float>(window_bytes) * (heter ? 1.f / 600.f : 1.f / 300.f));
  each = each < 2048.f ? 2048.f : each > 65536.f ? 65536.f : each;
  const uint64_t want = (pairs + static_cast<uint32_t>(each) - 1u) / static_cast<uint32_t>(each);
  return want < 1u ? 1u : want > launched ? launched : static_cast<uint32_t>(want);
}

// SELF: no list.  The matrix has at most kSelfListRows rows and every workgroup looks at all events itself
// (thread t at rows t, t + 1,024, ...: bit b of its mask is row 1,024 b + t; the active rows are numbered thread
// by thread, then bit by bit, the same in every workgroup), which saves the launch of the kernel that lists
// them.  Active rows without nonzeros are then among the numbered ones.
constexpr uint32_t kSelfListRows = 32u * kBinThreads;
typedef uint32_t row4_u32 __attribute__((ext_vector_type(4), aligned(4)));
template <typename F, bool HETER, bool SELF>
__global__ __launch_bounds__(kBinThreads) void active_rows_window_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    uint32_t n_row, uint32_t n_col, const uint32_t *__restrict__ active_count, const uint2 *__restrict__ active_list,
    uint32_t list_cap, void *__restrict__ partial, uint32_t *__restrict__ groups_out, const void *__restrict__ events,
    uint32_t event_width, uint32_t slices, uint32_t slice_cols) {
  // grid = producers launched * slices: an output wider than one window is taken in `slices` slices of slice_cols
  // columns by as many sets of workgroups, which all walk the active rows and keep what falls into their slice
  using A = typename std::conditional<HETER, double, uint32_t>::type;  // a window's accumulators
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  A *window = reinterpret_cast<A *>(smem_raw);
  __shared__ uint32_t s_ptr[kTileRows + 1];     // nonzeros of the tile's rows before row k
  __shared__ uint32_t s_start[kTileRows];       // first nonzero of row k in the matrix
  __shared__ uint32_t s_hint[kBinThreads + 1];
  __shared__ uint32_t s_wave[kBinThreads / kWave];
  __shared__ uint32_t s_mask[SELF ? kBinThreads : 1];        // SELF: the active rows among a thread's 32
  __shared__ uint32_t s_before[SELF ? kBinThreads + 1 : 1];  // SELF: active rows of the threads before
  constexpr int U = 4;
  constexpr uint32_t kRound = U * kBinThreads;
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  uint32_t total;
  if constexpr (SELF) {
    // (every load is issued, beyond the last row for that row again, and none sits in a branch: they are in
    // flight together)
    auto scan = [&](const auto *ev) {
      uint32_t found = 0;
#pragma unroll
      for (uint32_t b = 0; b < 32u; ++b) {
        const uint32_t r = b * kBinThreads + tid;
        const auto v = ev[r < n_row ? r : n_row - 1u];
        if (v != 0 && r < n_row) found |= 1u << b;
      }
      return found;
    };
    const uint32_t m = event_width == 1u   ? scan(static_cast<const uint8_t *>(events))
                       : event_width == 4u ? scan(static_cast<const float *>(events))
                                           : scan(static_cast<const double *>(events));
    s_mask[tid] = m;
    const uint32_t c = static_cast<uint32_t>(__popc(m));
    const uint32_t incl = wave_inclusive_scan_u32(c);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave[w];
    s_before[tid] = before + incl - c;
    if (tid == kBinThreads - 1) s_before[kBinThreads] = before + incl;
    __syncthreads();
    total = s_before[kBinThreads];
  } else {
    total = active_count[0] < list_cap ? active_count[0] : list_cap;  // (never beyond the list)
  }
  const uint32_t producers = window_event_producers(total, indptr[n_row], n_row, gridDim.x / slices,
                                                    n_col * static_cast<uint32_t>(sizeof(A)), HETER);
  const uint32_t p = blockIdx.x / slices, slice = blockIdx.x % slices;
  if (blockIdx.x == 0 && tid == 0) groups_out[0] = producers;  // (for the kernel that adds the windows)
  if (p >= producers) return;
  const uint32_t c_lo = slice * slice_cols;
  const uint32_t width = slices > 1u ? (n_col - c_lo < slice_cols ? n_col - c_lo : slice_cols) : n_col;
  for (uint32_t i = tid; i < width; i += kBinThreads) window[i] = A(0);
  const uint32_t lo = static_cast<uint32_t>(static_cast<uint64_t>(p) * total / producers);
  const uint32_t hi = static_cast<uint32_t>(static_cast<uint64_t>(p + 1) * total / producers);

  auto row_of = [&](uint32_t j, uint32_t a, uint32_t b) {  // largest k in [a, b] with s_ptr[k] <= j
    while (a < b) {
      const uint32_t mid = (a + b + 1u) >> 1;
      if (s_ptr[mid] <= j) a = mid;
      else b = mid - 1u;
    }
    return a;
  };

  for (uint32_t t0 = lo; t0 < hi; t0 += kTileRows) {
    const uint32_t rows = (hi - t0 < kTileRows) ? hi - t0 : kTileRows;
    __syncthreads();  // the previous tile is done with s_ptr / s_start (and the window is cleared)
    uint2 e = make_uint2(0u, 0u);
    if (tid < rows) {
      if constexpr (SELF) {
        const uint32_t idx = t0 + tid;
        uint32_t a = 0, b = kBinThreads - 1u;  // the thread that holds active row idx: the largest a with s_before[a] <= idx
        while (a < b) {
          const uint32_t mid = (a + b + 1u) >> 1;
          if (s_before[mid] <= idx) a = mid;
          else b = mid - 1u;
        }
        uint32_t mask = s_mask[a];
        for (uint32_t k = idx - s_before[a]; k != 0; --k) mask &= mask - 1u;
        const uint32_t r = (static_cast<uint32_t>(__ffs(static_cast<int>(mask))) - 1u) * kBinThreads + a;
        const uint32_t first = indptr[r];
        e = make_uint2(first, indptr[r + 1] - first);
      } else {
        e = active_list[t0 + tid];
      }
    }
    const uint32_t incl = wave_inclusive_scan_u32(e.y);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave[w];
    if (tid < rows) s_ptr[tid] = before + incl - e.y, s_start[tid] = e.x;
    if (tid == rows - 1u) s_ptr[rows] = before + incl;
    __syncthreads();
    const uint32_t j1 = s_ptr[rows];  // the tile's nonzeros, numbered from 0 (a row without nonzeros is never found by row_of)
    for (uint32_t seg = 0; seg < j1; seg += kSegment) {
      const uint32_t seg_end = (j1 - seg < kSegment) ? j1 : seg + kSegment;
      __syncthreads();  // the previous segment is done with s_hint
      {
        const uint32_t j = seg + (tid << kHintShift);
        s_hint[tid] = (j < seg_end) ? row_of(j, 0u, rows - 1u) : rows - 1u;
        if (tid == 0) s_hint[kBinThreads] = rows - 1u;
      }
      __syncthreads();
      for (uint32_t jb = seg; jb < seg_end; jb += kRound) {
        // A lane takes U consecutive nonzeros of the round: one search for the row of the first (LDS only), a
        // walk from there for the others, and where they lie in one listed row (all but the few that cross
        // into the next) one request for their columns and one for their weights.
        const uint32_t j0 = jb + U * tid;
        uint32_t at[U];
        {
          const uint32_t jc = j0 < seg_end ? j0 : seg_end - 1u;
          const uint32_t q = (jc - seg) >> kHintShift;
          uint32_t k = row_of(jc, s_hint[q], s_hint[q + 1]);
          uint32_t e = s_ptr[k + 1u];
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const uint32_t ju = j0 + u < seg_end ? j0 + u : seg_end - 1u;
            while (e <= ju) e = s_ptr[++k + 1u];  // (ends: ju < seg_end <= s_ptr[rows])
            at[u] = s_start[k] + (ju - s_ptr[k]);
          }
        }
        uint32_t col[U];
        F val[U];
        bool together = j0 + U <= seg_end;  // (the listed rows are in no order: every one of the U is compared)
#pragma unroll
        for (int u = 1; u < U; ++u) together = together && at[u] == at[0] + static_cast<uint32_t>(u);
        if (together) {
          if (slices == 1u) {  // (the arrays pass through once; with slices the other slices' workgroups want the lines too)
            load_consecutive(indices + at[0], col);
            if (HETER) load_consecutive(data + at[0], val);
          } else {
            const row4_u32 c4 = *reinterpret_cast<const row4_u32 *>(indices + at[0]);
            col[0] = c4.x, col[1] = c4.y, col[2] = c4.z, col[3] = c4.w;
            if (HETER) {
#pragma unroll
              for (int u = 0; u < U; ++u) val[u] = data[at[0] + u];
            }
          }
        } else {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            col[u] = indices[at[u]];
            if (HETER) val[u] = data[at[u]];
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t rel = col[u] - c_lo;  // (wraps below the slice; a column beyond the output: left out)
          if (j0 + u < seg_end && rel < width) {
            if constexpr (HETER) atomicAdd(&window[rel], static_cast<double>(val[u]));
            else atomicAdd(&window[rel], 1u);
          }
        }
      }
    }
  }
  __syncthreads();
  A *mine = static_cast<A *>(partial) + static_cast<size_t>(p) * n_col + c_lo;
  for (uint32_t i = tid; i < width; i += kBinThreads) mine[i] = window[i];
}

// y[c] = the sum of the windows of the workgroups that took part (their number: counters[1]), in a fixed order
// (weights: in float64, rounded once; a homogeneous weight: the sum of as many additions of the weight as
// the windows counted).  Sets the list's counter, counters[0], back to zero for the next call.
template <typename F, bool HETER>
__global__ __launch_bounds__(kSumCols * kSumSlices) void sum_active_windows_kernel(const void *__restrict__ partial,
                                                                                   F *__restrict__ y, uint32_t n_col,
                                                                                   uint32_t *__restrict__ counters,
                                                                                   const F *__restrict__ data) {
  using A = typename std::conditional<HETER, double, uint32_t>::type;
  using S = typename std::conditional<HETER, double, uint64_t>::type;
  const uint32_t groups = counters[1];
  if (blockIdx.x == 0 && threadIdx.x == 0) counters[0] = 0u;
  bool mine;
  const S total = sum_windows_of_column<S, A>(static_cast<const A *>(partial), n_col, groups, &mine);
  if (mine) {
    const uint32_t c = blockIdx.x * kSumCols + threadIdx.x % kSumCols;
    if constexpr (HETER) y[c] = static_cast<F>(total);
    else y[c] = repeated_sum<F>(data[0], total);
  }
}

// grid = n_win * slices * parts; workgroup (b, q, s) adds share s of window b's pairs (its 8 runs
// taken as one sequence) to the zeroed y.  A window wider than the 2^lds_shift float64 accumulators
// in LDS is cut into `slices` = 2^(shift - lds_shift) slices: the workgroups of slice q read the
// same pairs and keep those that fall into their slice.
// Homogeneous weight (HETER false): a run holds the pairs' columns only (4 bytes each).  ONE workgroup
// per window and slice counts them (32-bit integers in LDS, sixteen loads per lane in flight), adds
// what the producers counted in y itself because a run was full, and stores the sum of that many
// additions of the weight: the reference's bits whatever the order of arrival, with no further
// launch.  (Measured against several workgroups per window that add their counts to y and a kernel
// of its own for the sums: 100,000 x 100,000, 1e8 nnz, 0.1 % events 20 against 23 us, 5 % 52 against
// 48 us.  With little activity the rows are added to y as sums of the weight itself, which is exact
// too: additions of one value give the same bits in any order.)
template <typename F, bool HETER, typename I>
__global__ __launch_bounds__(kBinThreads) void add_window_runs_kernel(F *__restrict__ y, uint32_t n_col, uint32_t shift,
                                                                      uint32_t lds_shift, uint32_t parts, uint32_t cap,
                                                                      const BinPair<F> *__restrict__ pairs,
                                                                      const uint32_t *__restrict__ fill,
                                                                      uint32_t *__restrict__ reset,
                                                                      const F *__restrict__ data,
                                                                      const I *__restrict__ indices,
                                                                      const uint2 *__restrict__ active_list,
                                                                      const uint32_t *__restrict__ active_colbase) {
  constexpr bool heter = HETER;
  extern __shared__ __attribute__((aligned(8))) unsigned char smem_raw[];
  // (the caller's active-row counter, left at zero for the next call)
  if (reset != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *reset = 0u;
  double *window = reinterpret_cast<double *>(smem_raw);
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  constexpr uint32_t kWaves = kBinThreads / kWave;
  const uint32_t direct_rows = fill[kDirectWord];
  if (direct_rows != 0u) {
    // k waves per active row (all the grid's waves when the rows are few), dealt over the
    // workgroups first; wave `part` of a row takes every k-th group of 64 nonzeros
    const F w_homo = heter ? F(0) : data[0];
    const uint32_t total_waves = gridDim.x * kWaves;
    const uint32_t k = direct_rows < total_waves ? total_waves / direct_rows : 1u;
    const uint64_t items = static_cast<uint64_t>(direct_rows) * k;
    for (uint64_t item = wave * gridDim.x + blockIdx.x; item < items; item += total_waves) {
      const uint32_t r = static_cast<uint32_t>(item / k), part = static_cast<uint32_t>(item % k);
      const uint2 e = active_list[r];  // (first nonzero, length)
      F *out = y + (active_colbase ? active_colbase[r] : 0u);
      for (uint32_t j = part * kWave + lane; j < e.y; j += k * kWave)
        atomic_add(out + indices[e.x + j], heter ? data[e.x + j] : w_homo);
    }
    return;
  }
  const uint32_t slices = 1u << (shift - lds_shift);
  const uint32_t b = blockIdx.x / (parts * slices), q = (blockIdx.x / parts) % slices, s = blockIdx.x % parts;
  // pre[r] = pairs in the runs before run r (at most 2^27 in all)
  uint32_t pre[kSubRuns + 1];
  pre[0] = 0;
#pragma unroll
  for (uint32_t r = 0; r < kSubRuns; ++r) {
    uint32_t c = fill[(b * kSubRuns + r) * kFillStride];
    if (c > cap) c = cap;  // the producers count what they could not store too
    pre[r + 1] = pre[r] + c;
  }
  const uint32_t n = pre[kSubRuns];
  // every workgroup that takes part adds a whole window to y: few pairs, few workgroups
  const uint32_t want = (n + kPairsPerPart - 1u) / kPairsPerPart;
  if (want < parts) parts = want;
  if (!HETER && parts > 1u) parts = 1u;  // (the one workgroup that forms the window's sums from their counts)
  if (s >= parts) return;
  const uint32_t lo = static_cast<uint32_t>(static_cast<uint64_t>(s) * n / parts);
  const uint32_t hi = static_cast<uint32_t>(static_cast<uint64_t>(s + 1) * n / parts);
  const uint32_t r0 = q << lds_shift;  // first column of the slice within the window
  const uint32_t c0 = (b << shift) + r0;
  if (c0 >= n_col) return;
  const uint32_t width = (n_col - c0 < (1u << lds_shift)) ? n_col - c0 : (1u << lds_shift);
  const BinPair<F> *runs = pairs + static_cast<uint64_t>(b) * kSubRuns * cap;
  // pair number v of the window's runs taken as one sequence
  auto pair_at = [&](uint32_t v) -> const BinPair<F> & {
    uint32_t r = 0, first = 0;
#pragma unroll
    for (uint32_t k = 1; k < kSubRuns; ++k)
      if (v >= pre[k]) r = k, first = pre[k];
    return runs[static_cast<uint64_t>(r) * cap + (v - first)];
  };
  if constexpr (!HETER) {
    // run r of this window: columns[r * cap .. + its fill)
    const uint32_t *columns = reinterpret_cast<const uint32_t *>(pairs) + static_cast<uint64_t>(b) * kSubRuns * cap;
    auto column_at = [&](uint32_t v) {
      uint32_t r = 0, first = 0;
#pragma unroll
      for (uint32_t k = 1; k < kSubRuns; ++k)
        if (v >= pre[k]) r = k, first = pre[k];
      return columns[static_cast<uint64_t>(r) * cap + (v - first)];
    };
    uint32_t *cwindow = reinterpret_cast<uint32_t *>(smem_raw);
    for (uint32_t i = tid; i < width; i += kBinThreads) cwindow[i] = 0u;
    __syncthreads();
    constexpr int UC = 16;
    for (uint32_t i0 = lo + wave * (UC * kWave); i0 < hi; i0 += kWaves * UC * kWave) {
      uint32_t rel[UC];
      if (i0 + UC * kWave <= hi) {
#pragma unroll
        for (int u = 0; u < UC; ++u) rel[u] = column_at(i0 + u * kWave + lane);
      } else {
#pragma unroll
        for (int u = 0; u < UC; ++u) {
          const uint32_t v = i0 + u * kWave + lane;
          rel[u] = 0xffffffffu;
          if (v < hi) rel[u] = column_at(v);
        }
      }
#pragma unroll
      for (int u = 0; u < UC; ++u)
        if (rel[u] - r0 < width) atomicAdd(&cwindow[rel[u] - r0], 1u);  // (wraps below r0)
    }
    __syncthreads();
    const F w_homo = data[0];
    for (uint32_t i = tid; i < width; i += kBinThreads) {
      const uint64_t count = static_cast<uint64_t>(cwindow[i]) + synapse_count(y[c0 + i]);
      if (count != 0u) y[c0 + i] = repeated_sum<F>(w_homo, count);
    }
    return;
  }
  for (uint32_t i = tid; i < width; i += kBinThreads) window[i] = 0.0;
  __syncthreads();
  constexpr int U = 8;
  for (uint32_t i0 = lo + wave * (U * kWave); i0 < hi; i0 += kWaves * U * kWave) {
    BinPair<F> e[U];
    if (i0 + U * kWave <= hi) {  // full steps: plain loads, all in flight
#pragma unroll
      for (int u = 0; u < U; ++u) e[u] = pair_at(i0 + u * kWave + lane);
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = i0 + u * kWave + lane;
        e[u].rel = 0xffffffffu;
        e[u].val = F(0);
        if (v < hi) e[u] = pair_at(v);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (e[u].rel - r0 < width) atomicAdd(&window[e[u].rel - r0], static_cast<double>(e[u].val));  // (wraps below r0)
  }
  __syncthreads();
  for (uint32_t i = tid; i < width; i += kBinThreads) {
    const F v = static_cast<F>(window[i]);
    if (v != F(0)) atomic_add(y + c0 + i, v);
  }
}

// log2 of the output window with event input: as many windows as the 7-bit ids allow (every
// consumer workgroup adds a whole window to y, so small windows and few workgroups per window).
// Up to 2^14 columns a window has its accumulators in LDS at once; wider ones (outputs above two
// million columns) are added in slices of 2^14, each slice reading the window's pairs again.
inline uint32_t event_window_shift(uint32_t n_out) {
  uint32_t shift = 8;
  while (shift < kBinMaxShift && (n_out >> shift) >= kMaxWindows) ++shift;
  return shift;
}

// Pairs all windows' runs hold together.  The host knows neither the nonzero count nor the
// activity, and what does not fit goes through direct atomics at a fortieth of the speed, so the
// scratch memory is sized generously for this device: 4,096 pairs per row or column, between 2^24
// and 2^27 (1 GB of float pairs: every nonzero of a 1e8-nnz matrix active at once).
inline uint64_t event_run_pairs(uint32_t n_row, uint32_t n_col) {
  uint64_t t = 4096ull * (n_row > n_col ? n_row : n_col);
  if (t < (1ull << 24)) t = 1ull << 24;
  if (t > (1ull << 27)) t = 1ull << 27;
  return t;
}

}  // namespace

// Without a list the window shares the LDS with 8 KB of masks: 58 KB of it (7,424 float64 accumulators or
// 14,848 counts), and an output of up to two such windows of float64 is taken in slices.  (Three and four
// slices, every slice walking all active nonzeros: 20,000 columns gain 2 us at 5 % events and lose 5 at 20 %
// against the sorted scatter, 25,000 columns lose at both.)
constexpr size_t kSelfWindowBytes = 58 * 1024;
constexpr uint32_t kSelfMaxSlices = 2;
bool window_event_scatter_self_usable(uint32_t n_row, uint32_t n_col, bool heter) {
  // (a homogeneous weight: up to four slices of 14,848 integer counts, as with a list of the active rows below)
  const uint32_t widest = heter ? kSelfMaxSlices * static_cast<uint32_t>(kSelfWindowBytes / sizeof(double))
                                : 4u * static_cast<uint32_t>(kSelfWindowBytes / sizeof(uint32_t));
  return n_col != 0 && n_col <= widest && n_row != 0 && n_row <= kSelfListRows;
}

// A homogeneous weight counts synapses in 32-bit integers, 14,848 to a window of 58 KB, and an output of up to four
// such windows is taken in slices by as many sets of workgroups, which all walk the active rows (their indices
// come from the L2s after the first set's read): no pairs written and read back.  50,000 x 50,000 with 5,000 per
// row: 33 / 81 / 267 us through the sorted scatter at 1 / 5 / 20 % events, 30 / 54 / 139 us so; 50,000 x 20,000
// with 1,000 per row: 22 / 36 / 73 / 185 us at 1 / 5 / 20 / 60 % against 21 / 26 / 34 / 57 us.  Every workgroup
// that takes part leaves a window of the output's width behind, whatever the activity, which matrices of many
// short rows do not earn back at the 1 % of a quiet network (1,000,000 x 59,000 with 100 per row: 26 -> 34 us,
// and 175 -> 117 us at 30 %; the host knows the rows, not their lengths): up to 65,536 rows.  Weights per synapse
// (float64 accumulators, half as many to a window) gain only from 20 % activity on and stay with the sorted scatter.
constexpr uint32_t kListedHomoMaxSlices = 4;
constexpr uint32_t kListedHomoMaxRows = 65536;
template <typename F>
bool window_event_scatter_usable(uint32_t n_row, uint32_t n_col, bool heter) {
  if (n_col == 0 || n_row == 0) return false;
  if (n_col <= kWindowEventMaxCols) return true;
  return !heter && n_row <= kListedHomoMaxRows &&
         n_col <= kListedHomoMaxSlices * static_cast<uint32_t>(kSelfWindowBytes / sizeof(uint32_t));
}


// scratch memory (behind the list, if there is one): the windows of two workgroups per CU, or, of an output in
// slices, of as many as take a slice
template <typename F>
size_t window_event_scatter_bytes(uint32_t n_col) {
  const uint32_t resident = 2u * static_cast<uint32_t>(device_info().num_cu);
  // (the fewest slices an output of this width is taken in, those of 32-bit counts, and float64 accumulators:
  // enough for either kind of weight)
  const uint32_t slices = n_col <= kWindowEventMaxCols ? 1u : div_up(n_col, static_cast<uint32_t>(kSelfWindowBytes / sizeof(uint32_t)));
  return static_cast<size_t>(resident / slices) * n_col * sizeof(double);
}

template <typename F>
bool window_event_scatter(hipStream_t stream, const F *data, bool heter, const uint32_t *indices, const uint32_t *indptr,
                          F *y, uint32_t n_row, uint32_t n_col, uint32_t *counters, const uint2 *active_list,
                          uint32_t list_cap, void *scratch, size_t scratch_bytes, const void *events, uint32_t event_width) {
  const bool self = events != nullptr;  // no list: the kernel looks at the events itself
  if (self ? !window_event_scatter_self_usable(n_row, n_col, heter) : !window_event_scatter_usable<F>(n_row, n_col, heter)) return false;
  if (scratch_bytes < window_event_scatter_bytes<F>(n_col)) return false;
  if (self && event_width != 1u && event_width != 4u && event_width != 8u) return false;
  const size_t acc_bytes = heter ? sizeof(double) : sizeof(uint32_t);
  // (the masks beside 12.5 KB of row tables: two workgroups must still fit a CU's 160 KB)
  const bool sliced = self || n_col > kWindowEventMaxCols;
  const uint32_t slice_cols = sliced ? static_cast<uint32_t>(kSelfWindowBytes / acc_bytes) : n_col;
  const uint32_t slices = sliced ? div_up(n_col, slice_cols) : 1u;
  const unsigned launched = 2u * static_cast<unsigned>(device_info().num_cu) / slices;
  const unsigned grid = launched * slices;
  const size_t lds = static_cast<size_t>(slices > 1u ? slice_cols : n_col) * acc_bytes;
  using Kernel = void (*)(const F *, const uint32_t *, const uint32_t *, uint32_t, uint32_t, const uint32_t *, const uint2 *,
                          uint32_t, void *, uint32_t *, const void *, uint32_t, uint32_t, uint32_t);
  const Kernel kernel = heter ? (self ? active_rows_window_kernel<F, true, true> : active_rows_window_kernel<F, true, false>)
                              : (self ? active_rows_window_kernel<F, false, true> : active_rows_window_kernel<F, false, false>);
  static thread_local bool attr_set[2][2] = {{false, false}, {false, false}};
  if (!attr_set[heter][self]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(kWindowEventMaxCols * sizeof(double))) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set[heter][self] = true;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kBinThreads), lds, stream, data, indices, indptr, n_row, n_col,
                     static_cast<const uint32_t *>(counters), active_list, list_cap, scratch, counters + 1, events, event_width,
                     slices, slice_cols);
  if (heter)
    hipLaunchKernelGGL((sum_active_windows_kernel<F, true>), dim3(div_up(n_col, kSumCols)), dim3(kSumCols * kSumSlices), 0, stream,
                       static_cast<const void *>(scratch), y, n_col, counters, data);
  else
    hipLaunchKernelGGL((sum_active_windows_kernel<F, false>), dim3(div_up(n_col, kSumCols)), dim3(kSumCols * kSumSlices), 0, stream,
                       static_cast<const void *>(scratch), y, n_col, counters, data);
  return true;
}

template <typename F>
bool bin_event_scatter_usable(uint32_t n_col) {
  const uint32_t n_win = div_up(n_col, 1u << event_window_shift(n_col));
  return n_win >= 2 && n_win <= kMaxWindows;
}

template <typename F>
size_t bin_event_scatter_bytes(uint32_t n_row, uint32_t n_col) {
  const uint32_t n_win = div_up(n_col, 1u << event_window_shift(n_col));
  const uint64_t cap = event_run_pairs(n_row, n_col) / (n_win * kSubRuns);
  return kBinEventFillBytes + static_cast<size_t>(cap) * n_win * kSubRuns * sizeof(BinPair<F>);
}

// at least kMinRunPairs pairs per run
constexpr uint32_t kMinRunPairs = 1024;
template <typename F>
size_t bin_event_scatter_min_bytes(uint32_t n_col) {
  const uint32_t n_win = div_up(n_col, 1u << event_window_shift(n_col));
  return kBinEventFillBytes + static_cast<size_t>(kMinRunPairs) * n_win * kSubRuns * sizeof(BinPair<F>);
}

template <typename F, typename I>
bool bin_event_scatter(hipStream_t stream, const F *data, bool heter, const I *indices, const I *indptr,
                       F *y, uint32_t n_row, uint32_t n_col, uint32_t *active_count, const uint2 *active_list,
                       uint32_t list_cap, void *scratch, size_t scratch_bytes, const uint32_t *active_colbase) {
  const uint32_t shift = event_window_shift(n_col);
  const uint32_t n_win = div_up(n_col, 1u << shift);
  if (scratch_bytes < bin_event_scatter_min_bytes<F>(n_col)) return false;
  // pairs per run: what the scratch memory holds (a window's kSubRuns runs together stay below
  // 2^28 pairs, which the consumer counts in 32 bits)
  const uint64_t cap64 = (scratch_bytes - kBinEventFillBytes) / (static_cast<size_t>(n_win) * kSubRuns * sizeof(BinPair<F>));
  const uint64_t cap_max = (1ull << 28) / kSubRuns;
  const uint32_t cap = static_cast<uint32_t>(cap64 > cap_max ? cap_max : cap64);
  uint32_t *fill = static_cast<uint32_t *>(scratch);
  BinPair<F> *pairs = reinterpret_cast<BinPair<F> *>(static_cast<unsigned char *>(scratch) + kBinEventFillBytes);
  const unsigned num_cu = static_cast<unsigned>(device_info().num_cu);
  uint32_t parts = num_cu / n_win;
  if (parts == 0) parts = 1;
  auto add_kernel = heter ? add_window_runs_kernel<F, true, I> : add_window_runs_kernel<F, false, I>;
  const uint32_t lds_shift = bin_lds_shift(shift);
  const uint32_t slices = 1u << (shift - lds_shift);
  if (slices > 1) parts = 1;
  const size_t lds = sizeof(double) << lds_shift;
  static thread_local bool attr_set[2] = {false, false};  // (per instantiation: one pair for every index type)
  if (!attr_set[heter] && lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(add_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set[heter] = true;
  }
  const uint32_t producers = 2u * num_cu;
  if (heter)
    hipLaunchKernelGGL((bin_active_rows_kernel<F, true, I>), dim3(producers), dim3(kBinThreads), 0, stream, data, indices,
                       indptr, n_row, active_count, active_list, list_cap, active_colbase, y, shift, cap, pairs, fill);
  else
    hipLaunchKernelGGL((bin_active_rows_kernel<F, false, I>), dim3(producers), dim3(kBinThreads), 0, stream, data, indices,
                       indptr, n_row, active_count, active_list, list_cap, active_colbase, y, shift, cap, pairs, fill);
  hipLaunchKernelGGL(add_kernel, dim3(n_win * slices * parts), dim3(kBinThreads), lds, stream, y, n_col, shift,
                     lds_shift, parts, cap, pairs, fill, active_count, data, indices, active_list, active_colbase);
  return true;
}

template <typename F>
bool flat_window_scatter(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                         const uint32_t *indptr, const F *vec, F *y, uint32_t n_row, uint32_t n_col) {
  if (n_row == 0 || n_col == 0 || n_col > kFlatWindowMaxSlices * kFlatWindowMaxCols) return false;
  const uint32_t slices = div_up(n_col, kFlatWindowMaxCols);
  const size_t lds = static_cast<size_t>(slices > 1 ? kFlatWindowMaxCols : n_col) * sizeof(double);
  auto kernel = heter ? flat_window_kernel<F, true> : flat_window_kernel<F, false>;
  static thread_local bool attr_set[2] = {false, false};
  if (!attr_set[heter]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(kFlatWindowMaxCols * sizeof(double))) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set[heter] = true;
  }
  // two workgroups per CU where their windows and 12 KB of row tables each fit the CU's 160 KB
  const unsigned num_cu = static_cast<unsigned>(device_info().num_cu);
  const size_t static_lds = 2 * (kBinThreads + 1) * sizeof(uint32_t) + kTileRows * sizeof(F) + 256;  // (row tables)
  unsigned shares = (lds + static_lds <= 80 * 1024 ? 2u : 1u) * num_cu / slices;
  if (shares > div_up(n_row, 64)) shares = div_up(n_row, 64);
  const size_t partial_bytes = static_cast<size_t>(shares) * n_col * sizeof(double);
  double *partial = static_cast<double *>(stream_workspace(stream, partial_bytes));
  if (partial == nullptr) {
    if (!scratch_refused_by_capture()) bpl_clear_error();  // (an allocation failed: the caller has other paths)
    return false;
  }
  hipLaunchKernelGGL(kernel, dim3(shares * slices), dim3(kBinThreads), lds, stream, data, indices, indptr, vec, n_row,
                     n_col, slices, partial);
  hipLaunchKernelGGL(sum_windows_kernel<F>, dim3(div_up(n_col, kSumCols)), dim3(kSumCols * kSumSlices), 0, stream,
                     static_cast<const double *>(partial), y, n_col, shares);
  return check_launch(target);
}

constexpr uint64_t kChunkPairBytes = 200ull << 20;
constexpr uint32_t kMaxChunks = 6;

template <typename F>
bool bin_scatter_usable(uint32_t n_col, uint32_t nnz) {
  const uint32_t n_win = div_up(n_col, 1u << bin_window_shift(n_col));
  return n_win >= 2 && n_win <= kMaxWindows && nnz >= (1u << 20);
}

template <typename F>
bool bin_scatter(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                 const uint32_t *indptr, const F *vec, F *y, uint32_t n_row, uint32_t n_col, uint32_t nnz) {
  const uint32_t shift = bin_window_shift(n_col);
  const uint32_t n_win = div_up(n_col, 1u << shift);
  const unsigned num_cu = static_cast<unsigned>(device_info().num_cu);
  // two producer workgroups per CU, each an equal share of the nonzeros
  const uint32_t producers = 2u * num_cu;
  const uint32_t lds_shift = bin_lds_shift(shift);
  const uint32_t slices = 1u << (shift - lds_shift);
  uint32_t parts = num_cu / (n_win * slices);
  if (parts == 0) parts = 1;
  if (parts > producers) parts = producers;

  // the last region ends at or before nnz + nnz / 4 + producers * n_win * kRegionSpacing
  const bool packed = shift <= 16;
  const size_t n_pairs =
      (static_cast<size_t>(nnz) + nnz / 4u + static_cast<size_t>(producers) * n_win * kRegionSpacing + 127u) / 64u * 64u;
  const size_t pair_bytes = (n_pairs * bin_pair_bytes<F>(packed) + 255) / 256 * 256;
  const size_t count_bytes = static_cast<size_t>(n_win) * producers * sizeof(uint32_t);
  unsigned char *ws = static_cast<unsigned char *>(stream_workspace(stream, pair_bytes + count_bytes));
  if (ws == nullptr) {
    if (!scratch_refused_by_capture()) bpl_clear_error();  // (an allocation failed: the caller has other paths)
    return false;
  }
  void *pairs = ws;
  uint32_t *counts = reinterpret_cast<uint32_t *>(ws + pair_bytes);

  auto add_kernel = packed ? add_bins_kernel<F, true, false> : add_bins_kernel<F, false, false>;
  const size_t lds = sizeof(double) << lds_shift;
  static thread_local bool attr_set[2] = {false, false};
  if (!attr_set[packed] && lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(add_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set[packed] = true;
  }
  fill_zero(stream, y, n_col);
  auto bin_kernel = heter ? (packed ? bin_products_kernel<F, true, true> : bin_products_kernel<F, true, false>)
                          : (packed ? bin_products_kernel<F, false, true> : bin_products_kernel<F, false, false>);
  // The nonzeros are taken in chunks whose pairs (about kChunkPairBytes) stay in the 256 MB cache in front of the
  // memory between the kernel that writes them and the kernel that reads them: at 1e8 nonzeros three chunks
  // take 535 us, one 590, six 630 (every chunk is a pair of launches that start and drain on their own, and
  // one more float32 addition per output element).
  uint32_t chunks = div_up(static_cast<uint64_t>(nnz) * bin_pair_bytes<F>(packed), kChunkPairBytes);
  if (chunks > kMaxChunks) chunks = kMaxChunks;
  if (chunks == 0) chunks = 1;
  const uint32_t chunk_nnz = (div_up(nnz, chunks) + 3u) & ~3u;
  for (uint32_t c = 0; c < chunks; ++c) {
    const uint64_t lo = static_cast<uint64_t>(c) * chunk_nnz;
    if (lo >= nnz && c != 0) break;
    const uint32_t last = (c + 1 == chunks || lo + chunk_nnz >= nnz) ? 1u : 0u;
    hipLaunchKernelGGL(bin_kernel, dim3(producers), dim3(kBinThreads), 0, stream, data, indices, indptr, vec, y, n_row,
                       static_cast<uint32_t>(lo), chunk_nnz, last, n_win, shift, pairs, static_cast<uint64_t>(n_pairs), counts);
    hipLaunchKernelGGL(add_kernel, dim3(n_win * slices * parts), dim3(kBinThreads), lds, stream, indptr, y, n_row, n_col,
                       static_cast<uint32_t>(lo), chunk_nnz, last, n_win, shift, lds_shift, parts, producers,
                       static_cast<const void *>(pairs), static_cast<uint64_t>(n_pairs), counts, 0u,
                       static_cast<uint32_t *>(nullptr));
    if (last) break;
  }
  return check_launch(target);
}

// Adds uniformly laid out bins (filled by another producer, e.g. the jitconn column walk) to
// the zeroed y of n_out elements: bin (p, b) = pairs + (p * n_win + b) * cap with counts[b * producers + p] pairs.
template <typename F>
bool add_uniform_bins(const char *target, hipStream_t stream, F *y, uint32_t n_out, uint32_t shift, uint32_t producers,
                      uint32_t cap, const void *pairs, bool packed, const uint32_t *counts, uint32_t *reset) {
  const uint32_t n_win = div_up(n_out, 1u << shift);
  auto add_kernel = packed ? add_bins_kernel<F, true, true> : add_bins_kernel<F, false, false>;
  const uint32_t lds_shift = bin_lds_shift(shift);
  const uint32_t slices = 1u << (shift - lds_shift);
  const size_t lds = sizeof(double) << lds_shift;
  static thread_local bool attr_set[2] = {false, false};
  if (!attr_set[packed] && lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(add_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set[packed] = true;
  }
  uint32_t parts = static_cast<uint32_t>(device_info().num_cu) / (n_win * slices);
  if (parts == 0) parts = 1;
  if (parts > producers) parts = producers;
  const uint64_t n_pairs = static_cast<uint64_t>(producers) * n_win * cap;
  hipLaunchKernelGGL(add_kernel, dim3(n_win * slices * parts), dim3(kBinThreads), lds, stream,
                     static_cast<const uint32_t *>(nullptr), y, 0u, n_out, 0u, 0u, 0u, n_win, shift, lds_shift, parts, producers,
                     pairs, n_pairs, counts, cap, reset);
  return check_launch(target);
}

template bool add_uniform_bins<float>(const char *, hipStream_t, float *, uint32_t, uint32_t, uint32_t, uint32_t, const void *,
                                      bool, const uint32_t *, uint32_t *);
template bool add_uniform_bins<double>(const char *, hipStream_t, double *, uint32_t, uint32_t, uint32_t, uint32_t,
                                       const void *, bool, const uint32_t *, uint32_t *);
template bool window_event_scatter_usable<float>(uint32_t, uint32_t, bool);
template bool window_event_scatter_usable<double>(uint32_t, uint32_t, bool);
template size_t window_event_scatter_bytes<float>(uint32_t);
template size_t window_event_scatter_bytes<double>(uint32_t);
template bool window_event_scatter<float>(hipStream_t, const float *, bool, const uint32_t *, const uint32_t *, float *, uint32_t,
                                          uint32_t, uint32_t *, const uint2 *, uint32_t, void *, size_t, const void *, uint32_t);
template bool window_event_scatter<double>(hipStream_t, const double *, bool, const uint32_t *, const uint32_t *, double *,
                                           uint32_t, uint32_t, uint32_t *, const uint2 *, uint32_t, void *, size_t, const void *,
                                           uint32_t);
template bool bin_event_scatter_usable<float>(uint32_t);
template bool bin_event_scatter_usable<double>(uint32_t);
template size_t bin_event_scatter_bytes<float>(uint32_t, uint32_t);
template size_t bin_event_scatter_bytes<double>(uint32_t, uint32_t);
template size_t bin_event_scatter_min_bytes<float>(uint32_t);
template size_t bin_event_scatter_min_bytes<double>(uint32_t);
template bool bin_event_scatter<float, uint32_t>(hipStream_t, const float *, bool, const uint32_t *, const uint32_t *, float *,
                                                 uint32_t, uint32_t, uint32_t *, const uint2 *, uint32_t, void *, size_t,
                                                 const uint32_t *);
template bool bin_event_scatter<double, uint32_t>(hipStream_t, const double *, bool, const uint32_t *, const uint32_t *,
                                                  double *, uint32_t, uint32_t, uint32_t *, const uint2 *, uint32_t, void *,
                                                  size_t, const uint32_t *);
template bool bin_event_scatter<float, uint64_t>(hipStream_t, const float *, bool, const uint64_t *, const uint64_t *, float *,
                                                 uint32_t, uint32_t, uint32_t *, const uint2 *, uint32_t, void *, size_t,
                                                 const uint32_t *);
template bool bin_event_scatter<double, uint64_t>(hipStream_t, const double *, bool, const uint64_t *, const uint64_t *,
                                                  double *, uint32_t, uint32_t, uint32_t *, const uint2 *, uint32_t, void *,
                                                  size_t, const uint32_t *);
template bool flat_window_scatter<float>(const char *, hipStream_t, const float *, bool, const uint32_t *, const uint32_t *,
                                         const float *, float *, uint32_t, uint32_t);
template bool flat_window_scatter<double>(const char *, hipStream_t, const double *, bool, const uint32_t *,
                                          const uint32_t *, const double *, double *, uint32_t, uint32_t);
template bool bin_scatter_usable<float>(uint32_t, uint32_t);
template bool bin_scatter_usable<double>(uint32_t, uint32_t);
template bool bin_scatter<float>(const char *, hipStream_t, const float *, bool, const uint32_t *, const uint32_t *,
                                 const float *, float *, uint32_t, uint32_t, uint32_t);
template bool bin_scatter<double>(const char *, hipStream_t, const double *, bool, const uint32_t *, const uint32_t *,
                                  const double *, double *, uint32_t, uint32_t, uint32_t);

}  // namespace bpl
