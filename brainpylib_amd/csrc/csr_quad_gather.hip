// csr_matvec (no transpose) with the dense vector gathered from L2: the walk for vectors too long for LDS.
//
// Measured on this device: a product that reads one 4-byte element of a 4 MB vector per nonzero is bound
// by the rate at which a CU's vector cache takes misses (about one 128-byte line per 3.2 clocks and CU,
// whatever the occupancy), and the index and weight streams go through the same cache.  What helps is
// (a) fewer, wider stream requests: every lane loads FOUR consecutive nonzeros (16 bytes of indices, 16 or
// 32 bytes of weights) per request, (b) the nontemporal hint on the streams, so that the 800 MB that pass
// through do not push the vector out of the L2s, and (c) sixteen gathers in flight per lane.  A flat kernel
// without rows reaches 190-199 G nonzeros/s this way against 152-159 G/s with 4-byte stream loads; this walk
// reaches 160 G/s (lanes of a row's last step that lie beyond the row still cost their share of an instruction).
//
// Rows start anywhere, so a row is covered by the aligned quads [start / 4, ceil(end / 4)); the elements of
// its first and last quad that belong to the neighbouring rows are masked (their gather is pointed at
// element 0 of the vector).  G lanes walk the rows dealt to their group as one sequence of steps of 4 G
// quads: the quads of the next step, which may belong to the group's next row, are requested before this
// step's gathers are consumed.  G is chosen on the device from the mean row length.  Per-lane partial sums
// are float64, the product is formed in F first: the arithmetic of the reference's CPU loop
// (brainpylib/_src/sparse_ops/sparse_csr_matvec.py:116-119).
//
// Long rows: a row that would take its group more than 32 steps is not walked by the group; the row is
// noted in LDS and, after the walk, the whole workgroup takes the noted rows one by one (512 lanes, 16
// gathers each per step, partial sums combined in a fixed order).  The reference's kernel leaves such a
// row to one warp (lib/gpu_csr_matvec.cu:144-167).
#include "common.h"
#include "csr_quad_gather.h"

namespace bpl {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

// Two workgroups of 8 waves per CU (measured: 618 us for 1e8 nonzeros against 642 us with one of 16 waves,
// whose lanes have 128 registers and spill).
constexpr int kQuadThreads = 512;
constexpr unsigned kQuadPerCu = 2;
// quads per lane and step (U): 4 for float, 2 for double (registers)
constexpr uint32_t kLongSteps = 32;  // a row of more steps than this goes to the whole workgroup
constexpr uint32_t kMaxLong = 1024;  // rows a workgroup can note; further ones are walked by their group

template <typename F>
struct Quad {
  F v[4];
};

// Four consecutive indices / weights, quad q of the array (n elements).  Only the array's last quad can
// reach beyond its end: that one is read element by element.
__device__ __forceinline__ u32x4 load_index_quad(const uint32_t *__restrict__ p, uint32_t q, uint32_t n) {
  if (4u * q + 4u <= n) return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p) + q);
  u32x4 r = {0u, 0u, 0u, 0u};
  if (4u * q + 0u < n) r.x = p[4u * q + 0u];
  if (4u * q + 1u < n) r.y = p[4u * q + 1u];
  if (4u * q + 2u < n) r.z = p[4u * q + 2u];
  return r;
}
__device__ __forceinline__ Quad<float> load_data_quad(const float *__restrict__ p, uint32_t q, uint32_t n) {
  Quad<float> r = {{0.f, 0.f, 0.f, 0.f}};
  if (4u * q + 4u <= n) {
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p) + q);
    r.v[0] = v.x, r.v[1] = v.y, r.v[2] = v.z, r.v[3] = v.w;
  } else {
    for (uint32_t t = 0; t < 3; ++t)
      if (4u * q + t < n) r.v[t] = p[4u * q + t];
  }
  return r;
}
__device__ __forceinline__ Quad<double> load_data_quad(const double *__restrict__ p, uint32_t q, uint32_t n) {
  Quad<double> r = {{0., 0., 0., 0.}};
  if (4u * q + 4u <= n) {
    const f64x2 a = __builtin_nontemporal_load(reinterpret_cast<const f64x2 *>(p) + 2u * q);
    const f64x2 b = __builtin_nontemporal_load(reinterpret_cast<const f64x2 *>(p) + 2u * q + 1u);
    r.v[0] = a.x, r.v[1] = a.y, r.v[2] = b.x, r.v[3] = b.y;
  } else {
    for (uint32_t t = 0; t < 3; ++t)
      if (4u * q + t < n) r.v[t] = p[4u * q + t];
  }
  return r;
}

// One step of a lane: quads qfirst + u * stride (u < kQuadU) of the row [s, e), as far as they lie below qend.
template <typename F, bool HETER, int kQuadU>
struct Step {
  u32x4 ci[kQuadU];
  Quad<F> cd[kQuadU];

  __device__ __forceinline__ void load(const F *__restrict__ data, const uint32_t *__restrict__ indices, uint32_t nnz,
                                       uint32_t qfirst, uint32_t stride, uint32_t qend) {
#pragma unroll
    for (int u = 0; u < kQuadU; ++u) {
      const uint32_t q = qfirst + u * stride;
      ci[u] = u32x4{0u, 0u, 0u, 0u};
      if (q < qend) ci[u] = load_index_quad(indices, q, nnz);
    }
    if (HETER) {
#pragma unroll
      for (int u = 0; u < kQuadU; ++u) {
        const uint32_t q = qfirst + u * stride;
        cd[u] = Quad<F>{{F(0), F(0), F(0), F(0)}};
        if (q < qend) cd[u] = load_data_quad(data, q, nnz);
      }
    }
  }

  // bit 4 u + t: element t of quad u belongs to the row
  __device__ __forceinline__ uint32_t members(uint32_t qfirst, uint32_t stride, uint32_t s, uint32_t e) const {
    uint32_t m = 0;
#pragma unroll
    for (int u = 0; u < kQuadU; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t j = 4u * (qfirst + u * stride) + t;
        if (j >= s && j < e) m |= 1u << (4 * u + t);
      }
    }
    return m;
  }

  __device__ __forceinline__ void gather(const F *__restrict__ x, uint32_t m, F (&xv)[4 * kQuadU]) const {
#pragma unroll
    for (int u = 0; u < kQuadU; ++u) {
      const uint32_t c[4] = {ci[u].x, ci[u].y, ci[u].z, ci[u].w};
#pragma unroll
      for (int t = 0; t < 4; ++t) xv[4 * u + t] = x[((m >> (4 * u + t)) & 1u) ? c[t] : 0u];
    }
  }

  __device__ __forceinline__ double sum(uint32_t m, const F (&xv)[4 * kQuadU], F w_homo) const {
    double acc = 0.0;
#pragma unroll
    for (int u = 0; u < kQuadU; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // product formed in F, then widened (the reference multiplies two F values)
        const F p = static_cast<F>(xv[4 * u + t] * (HETER ? cd[u].v[t] : w_homo));
        acc += ((m >> (4 * u + t)) & 1u) ? static_cast<double>(p) : 0.0;
      }
    }
    return acc;
  }
};

template <typename F, bool HETER, int G, int kQuadU>
__device__ __forceinline__ void quad_walk(const F *__restrict__ data, const uint32_t *__restrict__ indices,
                                          const uint32_t *__restrict__ indptr, const F *__restrict__ x,
                                          F *__restrict__ y, uint32_t n_row, uint32_t nnz, uint32_t *s_long,
                                          uint32_t *s_long_count) {
  constexpr uint32_t kStepQuads = kQuadU * G;
  constexpr uint32_t kLong = kLongSteps * kStepQuads * 4u;  // nonzeros
  const uint32_t groups_per_block = kQuadThreads / G;
  const uint32_t gl = threadIdx.x % G;
  const uint32_t stride_rows = gridDim.x * groups_per_block;
  const F w_homo = HETER ? F(0) : data[0];

  // Bounds of `r` as the walk sees them: a long row is noted for the workgroup and looks empty here.
  auto classify = [&](uint32_t r, uint32_t &s, uint32_t &e, bool &store) {
    store = true;
    if (e - s > kLong) {
      uint32_t slot = 0;
      if (gl == 0) slot = atomicAdd(s_long_count, 1u);
      slot = __shfl(slot, static_cast<int>((threadIdx.x % kWave) - gl), kWave);
      if (slot < kMaxLong) {
        if (gl == 0) s_long[slot] = r;
        e = s;
        store = false;
      }
    }
  };

  uint32_t row = blockIdx.x * groups_per_block + threadIdx.x / G;
  bool have = row < n_row;
  uint32_t s = 0, e = 0, ns = 0, ne = 0;
  bool store = true;
  if (have) {
    s = indptr[row], e = indptr[row + 1];
    classify(row, s, e, store);
  }
  if (row + stride_rows < n_row) ns = indptr[row + stride_rows], ne = indptr[row + stride_rows + 1];
  uint32_t q = s >> 2, qe = e > s ? (e + 3u) >> 2 : q;

  Step<F, HETER, kQuadU> cur;
  if (have) cur.load(data, indices, nnz, q + gl, G, qe);
  double acc = 0.0;
  while (have) {
    const bool last = q + kStepQuads >= qe;
    uint32_t nrow = row, nq = q + kStepQuads, nqe = qe, nxs = s, nxe = e;
    bool nstore = store;
    if (last) {
      nrow = row + stride_rows;
      nxs = ns, nxe = ne;
      if (nrow < n_row) classify(nrow, nxs, nxe, nstore);
      nq = nxs >> 2, nqe = nxe > nxs ? (nxe + 3u) >> 2 : nq;
    }
    const bool more = nrow < n_row;

    const uint32_t m = cur.members(q + gl, G, s, e);
    F xv[4 * kQuadU];
    cur.gather(x, m, xv);
    Step<F, HETER, kQuadU> nxt;
    if (more) {
      nxt.load(data, indices, nnz, nq + gl, G, nqe);
      if (last && nrow + stride_rows < n_row)
        ns = indptr[nrow + stride_rows], ne = indptr[nrow + stride_rows + 1];
    }
    acc += cur.sum(m, xv, w_homo);
    if (last) {
      acc = group_sum<G>(acc);
      if (gl == 0 && store) y[row] = static_cast<F>(acc);
      acc = 0.0;
    }
    if (!more) break;
    row = nrow, q = nq, qe = nqe, s = nxs, e = nxe, store = nstore;
    cur = nxt;
  }
}

template <typename F, bool HETER>
__global__ __launch_bounds__(kQuadThreads) void csr_quad_gather_kernel(const F *__restrict__ data,
                                                                       const uint32_t *__restrict__ indices,
                                                                       const uint32_t *__restrict__ indptr,
                                                                       const F *__restrict__ x, F *__restrict__ y,
                                                                       uint32_t n_row, uint32_t min_mean) {
  __shared__ uint32_t s_long[kMaxLong];
  __shared__ uint32_t s_long_count;
  __shared__ double s_part[kQuadThreads / kWave];
  constexpr int kQuadU = sizeof(F) == 4 ? 4 : 2;
  const uint32_t nnz = indptr[n_row];
  const uint32_t mean = nnz / n_row;
  if (mean < min_mean) return;  // (the launcher's other kernel takes matrices of short rows)
  if (threadIdx.x == 0) s_long_count = 0;
  __syncthreads();
  if (mean >= 768) quad_walk<F, HETER, 64, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  else if (mean >= 384) quad_walk<F, HETER, 32, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  else if (mean >= 192) quad_walk<F, HETER, 16, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  else if (mean >= 80) quad_walk<F, HETER, 8, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  else if (mean >= 40) quad_walk<F, HETER, 4, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  else quad_walk<F, HETER, 2, kQuadU>(data, indices, indptr, x, y, n_row, nnz, s_long, &s_long_count);
  __syncthreads();

  // the rows noted as long: the whole workgroup, one row after the other
  const uint32_t n_long = s_long_count < kMaxLong ? s_long_count : kMaxLong;
  const F w_homo = HETER ? F(0) : data[0];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  for (uint32_t k = 0; k < n_long; ++k) {
    const uint32_t row = s_long[k];
    const uint32_t s = indptr[row], e = indptr[row + 1];
    const uint32_t qe = (e + 3u) >> 2;
    double acc = 0.0;
    for (uint32_t q = (s >> 2) + threadIdx.x; q < qe; q += kQuadU * kQuadThreads) {
      Step<F, HETER, kQuadU> st;
      st.load(data, indices, nnz, q, kQuadThreads, qe);
      const uint32_t m = st.members(q, kQuadThreads, s, e);
      F xv[4 * kQuadU];
      st.gather(x, m, xv);
      acc += st.sum(m, xv, w_homo);
    }
    acc = wave_sum(acc);
    if (lane == 0) s_part[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      double total = 0.0;
      for (uint32_t w = 0; w < kQuadThreads / kWave; ++w) total += s_part[w];
      y[row] = static_cast<F>(total);
    }
    __syncthreads();
  }
}

}  // namespace

template <typename F>
bool csr_quad_gather(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                     const uint32_t *indptr, const F *x, F *y, uint32_t n_row, uint32_t min_mean) {
  if (n_row == 0) return true;
  // 16-byte loads of the streams
  if ((reinterpret_cast<uintptr_t>(indices) & 15u) != 0 || (heter && (reinterpret_cast<uintptr_t>(data) & 15u) != 0))
    return false;
  const unsigned resident = static_cast<unsigned>(device_info().num_cu) * kQuadPerCu;
  const unsigned needed = div_up(n_row, kQuadThreads / kWave);
  const unsigned grid = needed < resident ? needed : resident;
  if (heter)
    hipLaunchKernelGGL((csr_quad_gather_kernel<F, true>), dim3(grid), dim3(kQuadThreads), 0, stream, data, indices, indptr,
                       x, y, n_row, min_mean);
  else
    hipLaunchKernelGGL((csr_quad_gather_kernel<F, false>), dim3(grid), dim3(kQuadThreads), 0, stream, data, indices,
                       indptr, x, y, n_row, min_mean);
  return check_launch(target);
}

template bool csr_quad_gather<float>(const char *, hipStream_t, const float *, bool, const uint32_t *, const uint32_t *,
                                     const float *, float *, uint32_t, uint32_t);
template bool csr_quad_gather<double>(const char *, hipStream_t, const double *, bool, const uint32_t *,
                                      const uint32_t *, const double *, double *, uint32_t, uint32_t);

}  // namespace bpl
