// csr_matvec (no transpose) with the dense vector gathered from L2, walked FLAT: every wave owns a contiguous
// range of the nonzeros, whatever rows they belong to, so that every lane of every load and gather carries a
// nonzero.  (A row-wise walk, groups of lanes taking whole rows in steps of 16-byte loads, pads each row to
// whole steps of its group: with 100 nonzeros per row a fifth of the lanes of its gather instructions lie
// beyond the row, and a gather instruction costs the address unit the same whether its lanes are masked or
// not.  That walk took 633 us at 1e8 nonzeros in rows of 100, this one 570; rows of 30: 449 against 315.)
//
// Measured on this device: a product that reads one 4-byte element of a 4 MB vector per nonzero is bound by
// the rate at which a CU's vector cache takes misses (about one 128-byte line per 3.2 clocks and CU, whatever
// the occupancy), and the index and weight streams go through the same cache.  What helps is fewer, wider
// stream requests (every lane loads FOUR consecutive nonzeros, 16 bytes of indices and 16 or 32 of weights,
// per request), the nontemporal hint on the streams, so that the 800 MB that pass through do not push the
// vector out of the L2s, and sixteen gathers in flight per lane.
//
// A wave takes its range in steps of U * 64 quads (1,024 nonzeros of float, 512 of double): 16-byte loads of
// the index and weight streams (nontemporal), sixteen gathers per lane, the products formed in F and widened
// as the reference's CPU loop does (brainpylib/_src/sparse_ops/sparse_csr_matvec.py:116-119).  Which row a
// nonzero belongs to comes from a window of 65 consecutive entries of indptr in LDS, beginning at the row the
// step begins in: a six-step search per quad, then a walk over the quad's four elements.  A lane adds a run of
// elements of one row to that row's float64 accumulator in LDS with one atomic.  Rows that end inside the step
// are stored; the partial sum of the row that is still open moves to accumulator 0 of the next step.  A step
// that meets more than 64 rows (empty rows, very short ones) takes further windows over the same registers.
//
// Rows across the ranges of two or more waves: a wave never stores a row that began before its range; it
// leaves that row's partial sum in head[wave], and the partial sum of the row still open at the end of its
// range in tail[wave] with the row's number.  A second, small kernel adds tail[w] and the heads of the waves
// that follow, up to the wave the row ends in, and stores the row.  Both arrays hold one entry per wave of the
// launch (the nonzero count is known on the device only; the number of waves is the launcher's).
#include "common.h"
#include "csr_flat_gather.h"

namespace bpl {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

constexpr int kFlatThreads = 512;
constexpr int kFlatWaves = kFlatThreads / kWave;
constexpr unsigned kFlatPerCu = 2;
constexpr uint32_t kFlatRows = 64;  // rows of an indptr window (one per lane)
constexpr uint32_t kNoRow = 0xffffffffu;

template <typename F>
struct FlatQuads {
  static constexpr int value = sizeof(F) == 4 ? 4 : 2;  // quads per lane and step (registers)
};

// quads a wave owns: the same on the device (both kernels) from the nonzero count and the number of waves
__device__ __forceinline__ uint32_t flat_quads_per_wave(uint32_t nnz, uint32_t waves, uint32_t step_quads) {
  const uint32_t quads = nnz / 4u + (nnz % 4u ? 1u : 0u);
  const uint32_t per = quads / waves + (quads % waves ? 1u : 0u);
  return (per + step_quads - 1u) / step_quads * step_quads;
}

// Four consecutive indices / weights, quad q of the array (n elements).  Only the array's last quad can
// reach beyond its end: that one is read element by element.
__device__ __forceinline__ u32x4 flat_index_quad(const uint32_t *__restrict__ p, uint32_t q, uint32_t n) {
  if (4u * q + 4u <= n) return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p) + q);
  u32x4 r = {0u, 0u, 0u, 0u};
  if (4u * q + 0u < n) r.x = p[4u * q + 0u];
  if (4u * q + 1u < n) r.y = p[4u * q + 1u];
  if (4u * q + 2u < n) r.z = p[4u * q + 2u];
  return r;
}
__device__ __forceinline__ void flat_data_quad(const float *__restrict__ p, uint32_t q, uint32_t n, float (&v)[4]) {
  if (4u * q + 4u <= n) {
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p) + q);
    v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
  } else {
    for (uint32_t t = 0; t < 4; ++t) v[t] = (4u * q + t < n) ? p[4u * q + t] : 0.f;
  }
}
__device__ __forceinline__ void flat_data_quad(const double *__restrict__ p, uint32_t q, uint32_t n, double (&v)[4]) {
  if (4u * q + 4u <= n) {
    const f64x2 a = __builtin_nontemporal_load(reinterpret_cast<const f64x2 *>(p) + 2u * q);
    const f64x2 b = __builtin_nontemporal_load(reinterpret_cast<const f64x2 *>(p) + 2u * q + 1u);
    v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
  } else {
    for (uint32_t t = 0; t < 4; ++t) v[t] = (4u * q + t < n) ? p[4u * q + t] : 0.;
  }
}

// The last row r in [0, n_row) with indptr[r] <= pos, for pos < indptr[n_row]: the wave searches together,
// 64 probes a round (four rounds for a million rows).
__device__ __forceinline__ uint32_t flat_row_of(const uint32_t *__restrict__ indptr, uint32_t n_row, uint32_t pos,
                                                uint32_t lane) {
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

template <typename F, bool HETER>
__global__ __launch_bounds__(kFlatThreads, 4) void csr_flat_gather_kernel(
    const F *__restrict__ data, const uint32_t *__restrict__ indices, const uint32_t *__restrict__ indptr,
    const F *__restrict__ x, F *__restrict__ y, uint32_t n_row, uint32_t min_mean, uint32_t max_mean,
    double *__restrict__ head, double *__restrict__ tail, uint32_t *__restrict__ tail_row) {
  constexpr int U = FlatQuads<F>::value;
  constexpr uint32_t kStepQuads = U * kWave;
  __shared__ uint32_t s_ptr_all[kFlatWaves][kFlatRows + 2];  // (entry 65: a sentinel)
  __shared__ double s_sum_all[kFlatWaves][kFlatRows];
  const uint32_t nnz = indptr[n_row];
  const uint32_t mean = nnz / n_row;
  if (mean < min_mean || mean >= max_mean || nnz > kFlatMaxNnz) return;  // (the launcher's other kernel takes those matrices)
  const uint32_t lane = static_cast<uint32_t>(lane_id()), wv = threadIdx.x / kWave;
  uint32_t *s_ptr = s_ptr_all[wv];
  double *s_sum = s_sum_all[wv];
  const uint32_t waves = gridDim.x * kFlatWaves, w = blockIdx.x * kFlatWaves + wv;
  const uint32_t per = flat_quads_per_wave(nnz, waves, kStepQuads);
  if (lane == 0) head[w] = 0.0, tail[w] = 0.0, tail_row[w] = kNoRow;
  const uint64_t first_quad = static_cast<uint64_t>(w) * per;
  if (4u * first_quad >= nnz) return;
  const uint32_t begin = static_cast<uint32_t>(4u * first_quad);  // the wave owns the nonzeros [begin, end)
  const uint32_t end = (4u * (first_quad + per) < nnz) ? static_cast<uint32_t>(4u * (first_quad + per)) : nnz;
  const F w_homo = HETER ? F(0) : data[0];

  // Invariant at the start of a step [s0, s1): r is the row that holds nonzero s0 or begins there (rows that
  // end at s0 or before are stored or left to the wave before); s_sum[0] holds what row r has gathered in
  // this wave so far, s_sum[1..63] are zero.  Wave 0 begins at row 0, so that leading empty rows are stored.
  uint32_t r = (w == 0) ? 0u : flat_row_of(indptr, n_row, begin, lane);
  s_sum[lane] = 0.0;
  if (lane == 0) s_ptr[kFlatRows + 1] = 0xffffffffu;

  // Two steps are under way at a time: the index and weight streams of step i + 1 are requested before the
  // gathers of step i are consumed (568 against 609 us at 1e8 nonzeros).  A step's window of indptr is
  // requested first of all: waiting for a load means waiting for every load issued before it.  (Keeping the
  // next step's gathers in flight as well needs more registers than two workgroups per CU leave: the
  // compiler spills, and a reloaded register is a load that waits for every gather before it: 750 us.)
  constexpr uint32_t kStep = 4u * kStepQuads;
  auto load_streams = [&](uint32_t s0, u32x4 (&ci)[U], F (&cd)[U][4]) {  // lane l: quads s0 / 4 + l, + 64, ...
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t q = s0 / 4u + static_cast<uint32_t>(u) * kWave + lane;
      ci[u] = u32x4{0u, 0u, 0u, 0u};
      if (s0 < end && 4u * q < end) ci[u] = flat_index_quad(indices, q, nnz);
    }
    if (HETER) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t q = s0 / 4u + static_cast<uint32_t>(u) * kWave + lane;
#pragma unroll
        for (int t = 0; t < 4; ++t) cd[u][t] = F(0);
        if (s0 < end && 4u * q < end) flat_data_quad(data, q, nnz, cd[u]);
      }
    }
  };
  u32x4 ci[U];
  F cd[U][4];
  load_streams(begin, ci, cd);
  for (uint32_t s0 = begin; s0 < end; s0 += kStep) {
    const uint32_t s1 = (end - s0 > kStep) ? s0 + kStep : end;
    uint32_t ptr_lane, ptr_last;
    auto load_window = [&]() {
      const uint64_t k = static_cast<uint64_t>(r) + lane;
      ptr_lane = k <= n_row ? indptr[k] : 0xffffffffu;
      ptr_last = static_cast<uint64_t>(r) + kFlatRows <= n_row ? indptr[r + kFlatRows] : 0xffffffffu;  // (one address: a broadcast)
    };
    load_window();
    F prod[U][4];  // (the vector's elements first, then the products: in F, as the reference forms them)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t p0 = 4u * (s0 / 4u + static_cast<uint32_t>(u) * kWave + lane);
      const uint32_t c[4] = {ci[u].x, ci[u].y, ci[u].z, ci[u].w};
#pragma unroll
      for (int t = 0; t < 4; ++t) prod[u][t] = x[(p0 + t < s1) ? c[t] : 0u];  // (beyond the step: element 0, unused)
    }
    F cw[U][4];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t) cw[u][t] = HETER ? cd[u][t] : w_homo;
    }
    load_streams(s1, ci, cd);  // (a step at or beyond the end of the range loads nothing)
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t) prod[u][t] = static_cast<F>(prod[u][t] * cw[u][t]);
    }
    // windows of 64 rows from r on, until one reaches beyond the step
    for (;;) {
      s_ptr[lane] = ptr_lane;
      if (lane == 0) s_ptr[kFlatRows] = ptr_last;
      __builtin_amdgcn_wave_barrier();
      const uint32_t lo = s_ptr[0], hi = ptr_last;  // this window takes the nonzeros [lo, hi) of the step
      // The row of every quad's first nonzero and the ends of that row and of the next one, for the U quads
      // together (the LDS reads of different quads do not wait for each other); then, without a branch, the
      // quads that lie in one row or in two; a loop only for quads that meet three rows or more.
      uint32_t kq[U], e1[U], e2[U];
#pragma unroll
      for (int u = 0; u < U; ++u) kq[u] = 0;  // the last k < 64 with s_ptr[k] <= max(p0, lo) (s_ptr[0] = lo)
#pragma unroll
      for (uint32_t step = kFlatRows / 2; step != 0; step >>= 1) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t p0 = 4u * (s0 / 4u + static_cast<uint32_t>(u) * kWave + lane);
          const uint32_t pe = p0 > lo ? p0 : lo;
          if (s_ptr[kq[u] + step] <= pe) kq[u] += step;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) e1[u] = s_ptr[kq[u] + 1u], e2[u] = s_ptr[kq[u] + 2u];  // (s_ptr[65] is a sentinel)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t p0 = 4u * (s0 / 4u + static_cast<uint32_t>(u) * kWave + lane);
        const uint32_t top = hi < s1 ? hi : s1;  // the window takes the nonzeros [lo, top)
        if (e2[u] > p0 + 3u || e1[u] >= top) {
          // one row, or two (what lies at e1 or behind belongs to row k + 1, unless that is the next window's)
          double acc0 = 0.0, acc1 = 0.0;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const uint32_t p = p0 + static_cast<uint32_t>(t);
            const double v = (p >= lo && p < top) ? static_cast<double>(prod[u][t]) : 0.0;
            acc0 += p < e1[u] ? v : 0.0;
            acc1 += p < e1[u] ? 0.0 : v;
          }
          if (acc0 != 0.0) atomicAdd(&s_sum[kq[u]], acc0);
          if (acc1 != 0.0) atomicAdd(&s_sum[kq[u] + 1u], acc1);
        } else if (p0 < top && p0 + 3u >= lo) {
          uint32_t k = kq[u];
          double acc = 0.0;
          uint32_t kacc = k;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const uint32_t p = p0 + static_cast<uint32_t>(t);
            if (p >= lo && p < top) {
              while (s_ptr[k + 1u] <= p) ++k;  // (ends below 64: p < hi = s_ptr[64])
              if (k != kacc) {
                if (acc != 0.0) atomicAdd(&s_sum[kacc], acc);
                acc = 0.0, kacc = k;
              }
              acc += static_cast<double>(prod[u][t]);
            }
          }
          if (acc != 0.0) atomicAdd(&s_sum[kacc], acc);
        }
      }
      __builtin_amdgcn_wave_barrier();
      // rows of the window that end inside the step (a prefix of the window): stored, or, the one that began
      // before this wave's range, left in head[]
      const uint64_t row = static_cast<uint64_t>(r) + lane;
      const bool ended = row < n_row && s_ptr[lane + 1u] <= s1;
      const uint32_t n_ended = static_cast<uint32_t>(__popcll(__ballot(ended)));
      if (ended) {
        const double total = s_sum[lane];
        if (w != 0 && ptr_lane < begin) head[w] = total;
        else y[row] = static_cast<F>(total);
      }
      const double open = n_ended < kFlatRows ? s_sum[n_ended] : 0.0;  // (wave uniform address: a broadcast)
      __builtin_amdgcn_wave_barrier();
      s_sum[lane] = 0.0;
      r += n_ended;
      if (n_ended < kFlatRows || r >= n_row) {
        if (lane == 0) s_sum[0] = open;
        break;
      }
      load_window();
    }
    __builtin_amdgcn_wave_barrier();
  }
  // the row that is still open at the end of the range (if it has nonzeros in it)
  if (lane == 0 && r < n_row) {
    const uint32_t rs = indptr[r];
    if (rs < end) {
      if (w != 0 && rs < begin) head[w] = s_sum[0];
      else tail[w] = s_sum[0], tail_row[w] = r;
    }
  }
}

// One wave per wave of the walk: the row left open at the end of range w = its tail + the heads of the ranges
// it runs through, in a fixed order.
template <typename F>
__global__ __launch_bounds__(kWave) void csr_flat_finish_kernel(const uint32_t *__restrict__ indptr, F *__restrict__ y,
                                                                uint32_t n_row, uint32_t min_mean, uint32_t max_mean,
                                                                uint32_t waves, const double *__restrict__ head,
                                                                const double *__restrict__ tail,
                                                                const uint32_t *__restrict__ tail_row) {
  constexpr uint32_t kStepQuads = FlatQuads<F>::value * kWave;
  const uint32_t nnz = indptr[n_row];
  const uint32_t mean = nnz / n_row;
  if (mean < min_mean || mean >= max_mean || nnz > kFlatMaxNnz) return;
  const uint32_t w = blockIdx.x, lane = threadIdx.x;
  const uint32_t row = tail_row[w];
  if (row == kNoRow) return;
  const uint32_t per = flat_quads_per_wave(nnz, waves, kStepQuads);
  const uint32_t last = ((indptr[row + 1u] - 1u) / 4u) / per;  // the range the row's last nonzero lies in
  double acc = 0.0;
  for (uint32_t v = w + 1u + lane; v <= last && v < waves; v += kWave) acc += head[v];
  acc = wave_sum(acc);
  if (lane == 0) y[row] = static_cast<F>(tail[w] + acc);
}

}  // namespace

template <typename F>
FlatGather csr_flat_gather(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                     const uint32_t *indptr, const F *x, F *y, uint32_t n_row, uint32_t min_mean, uint32_t max_mean) {
  if (n_row == 0) return FlatGather::kEnqueued;
  // 16-byte loads of the streams
  if ((reinterpret_cast<uintptr_t>(indices) & 15u) != 0 || (heter && (reinterpret_cast<uintptr_t>(data) & 15u) != 0))
    return FlatGather::kNotApplicable;
  const unsigned grid = static_cast<unsigned>(device_info().num_cu) * kFlatPerCu;
  const uint32_t waves = grid * kFlatWaves;
  // [head: waves doubles][tail: waves doubles][tail_row: waves words]
  unsigned char *ws = static_cast<unsigned char *>(stream_workspace(stream, static_cast<size_t>(waves) * 20u));
  if (ws == nullptr) return FlatGather::kFailed;
  double *head = reinterpret_cast<double *>(ws), *tail = head + waves;
  uint32_t *tail_row = reinterpret_cast<uint32_t *>(tail + waves);
  if (heter)
    hipLaunchKernelGGL((csr_flat_gather_kernel<F, true>), dim3(grid), dim3(kFlatThreads), 0, stream, data, indices, indptr,
                       x, y, n_row, min_mean, max_mean, head, tail, tail_row);
  else
    hipLaunchKernelGGL((csr_flat_gather_kernel<F, false>), dim3(grid), dim3(kFlatThreads), 0, stream, data, indices,
                       indptr, x, y, n_row, min_mean, max_mean, head, tail, tail_row);
  hipLaunchKernelGGL(csr_flat_finish_kernel<F>, dim3(waves), dim3(kWave), 0, stream, indptr, y, n_row, min_mean, max_mean,
                     waves, static_cast<const double *>(head), static_cast<const double *>(tail),
                     static_cast<const uint32_t *>(tail_row));
  return check_launch(target) ? FlatGather::kEnqueued : FlatGather::kFailed;
}

template FlatGather csr_flat_gather<float>(const char *, hipStream_t, const float *, bool, const uint32_t *, const uint32_t *,
                                     const float *, float *, uint32_t, uint32_t, uint32_t);
template FlatGather csr_flat_gather<double>(const char *, hipStream_t, const double *, bool, const uint32_t *,
                                      const uint32_t *, const double *, double *, uint32_t, uint32_t, uint32_t);

}  // namespace bpl
