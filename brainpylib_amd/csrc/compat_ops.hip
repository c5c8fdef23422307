// The older operator family of the reference that its models still call through
// brainpylib/_src/compat: csr_event_sum with 64-bit indices, coo_event_sum and coo_atomic_sum
// (lib/gpu_event_sum.cu, lib/gpu_atomic_sum.cu).  Same target names, buffer order and 8-byte
// descriptors.  These are thin kernels: one lane per connection (or one wave per active
// row), global atomics into the zeroed result.  csr_event_sum with 32-bit indices is the
// event_csr_matvec scatter and lives with it in csr_ops.hip.
//
// The product twins coo_atomic_prod and csr_event_prod multiply into a result of ones, as the
// reference's CPU kernels do (lib/cpu_atomic_prod.cc:5-43, lib/cpu_event_prod.cc:5-55).  The
// reference's GPU kernels of coo_atomic_prod (lib/gpu_atomic_prod.cu:26-98) set every BYTE of the
// result to 1 and then ADD; that is not followed.  It registers no GPU csr_event_prod although its
// Python layer names one (brainpylib/_src/compat/event_prod.py:107-127); those eight targets
// exist here under the names that layer builds.
#include "common.h"

namespace bpl {
namespace {

constexpr int kThreads = 256;

// One wave per row: active rows add their nonzeros into the result.
// only_from_2_32: the kernel runs only if the matrix has 2^32 nonzeros or more (it follows the sorted
// scatter, which leaves such a matrix alone).
template <typename F, typename I, bool HETER>
__global__ __launch_bounds__(kThreads) void csr_event_sum_kernel(const uint8_t *__restrict__ events,
                                                                 const I *__restrict__ indices,
                                                                 const I *__restrict__ indptr,
                                                                 const F *__restrict__ values,
                                                                 F *__restrict__ result, uint32_t pre_size,
                                                                 bool only_from_2_32) {
  if (only_from_2_32 && (static_cast<uint64_t>(indptr[pre_size]) >> 32) == 0) return;
  const uint32_t waves = gridDim.x * (kThreads / kWave);
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const F w_homo = HETER ? F(0) : values[0];
  for (uint32_t r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave; r < pre_size; r += waves) {
    if (events[r] == 0) continue;
    const uint64_t start = static_cast<uint64_t>(indptr[r]), end = static_cast<uint64_t>(indptr[r + 1]);
    for (uint64_t j = start + lane; j < end; j += kWave)
      atomic_add(result + static_cast<uint64_t>(indices[j]), HETER ? values[j] : w_homo);
  }
}

// One lane per connection: result[post_ids[i]] += value if events[pre_ids[i]].
template <typename F, typename I, bool HETER>
__global__ __launch_bounds__(kThreads) void coo_event_sum_kernel(const uint8_t *__restrict__ events,
                                                                 const I *__restrict__ pre_ids,
                                                                 const I *__restrict__ post_ids,
                                                                 const F *__restrict__ values,
                                                                 F *__restrict__ result, uint32_t conn_size) {
  const F w_homo = HETER ? F(0) : values[0];
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < conn_size; i += gridDim.x * kThreads) {
    if (events[static_cast<uint64_t>(pre_ids[i])] != 0)
      atomic_add(result + static_cast<uint64_t>(post_ids[i]), HETER ? values[i] : w_homo);
  }
}

// One lane per connection: result[post_ids[i]] += values[pre_ids[i]] (heter) or values[0] (homo).
template <typename F, typename I, bool HETER>
__global__ __launch_bounds__(kThreads) void coo_atomic_sum_kernel(const F *__restrict__ values,
                                                                  const I *__restrict__ post_ids,
                                                                  const I *__restrict__ pre_ids,
                                                                  F *__restrict__ result, uint32_t conn_size) {
  const F w_homo = HETER ? F(0) : values[0];
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < conn_size; i += gridDim.x * kThreads)
    atomic_add(result + static_cast<uint64_t>(post_ids[i]),
               HETER ? values[static_cast<uint64_t>(pre_ids[i])] : w_homo);
}

// *p *= v, atomically: compare-and-swap on the bit pattern (integer compare, so a NaN in the
// result cannot keep the loop going).  Lanes that meet on one address take turns.
__device__ __forceinline__ void atomic_mul(float *p, float v) {
  unsigned int *a = reinterpret_cast<unsigned int *>(p);
  unsigned int seen = __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), expected;
  do {
    expected = seen;
    seen = atomicCAS(a, expected, __float_as_uint(__uint_as_float(expected) * v));
  } while (seen != expected);
}
__device__ __forceinline__ void atomic_mul(double *p, double v) {
  unsigned long long *a = reinterpret_cast<unsigned long long *>(p);
  unsigned long long seen = __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), expected;
  do {
    expected = seen;
    seen = atomicCAS(a, expected,
                     static_cast<unsigned long long>(__double_as_longlong(__longlong_as_double(expected) * v)));
  } while (seen != expected);
}

template <typename F>
__global__ __launch_bounds__(kThreads) void fill_one_kernel(F *__restrict__ p, uint32_t n) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = F(1);
}

// One lane per connection: result[post_ids[i]] *= values[pre_ids[i]] (heter) or values[0] (homo).
template <typename F, typename I, bool HETER>
__global__ __launch_bounds__(kThreads) void coo_atomic_prod_kernel(const F *__restrict__ values,
                                                                   const I *__restrict__ post_ids,
                                                                   const I *__restrict__ pre_ids,
                                                                   F *__restrict__ result, uint32_t conn_size) {
  const F w_homo = HETER ? F(1) : values[0];
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < conn_size; i += gridDim.x * kThreads)
    atomic_mul(result + static_cast<uint64_t>(post_ids[i]),
               HETER ? values[static_cast<uint64_t>(pre_ids[i])] : w_homo);
}

// One wave per row: active rows multiply their nonzeros into the result.
template <typename F, typename I, bool HETER>
__global__ __launch_bounds__(kThreads) void csr_event_prod_kernel(const uint8_t *__restrict__ events,
                                                                  const I *__restrict__ indices,
                                                                  const I *__restrict__ indptr,
                                                                  const F *__restrict__ values,
                                                                  F *__restrict__ result, uint32_t pre_size) {
  const uint32_t waves = gridDim.x * (kThreads / kWave);
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const F w_homo = HETER ? F(1) : values[0];
  for (uint32_t r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave; r < pre_size; r += waves) {
    if (events[r] == 0) continue;
    const uint64_t start = static_cast<uint64_t>(indptr[r]), end = static_cast<uint64_t>(indptr[r + 1]);
    for (uint64_t j = start + lane; j < end; j += kWave)
      atomic_mul(result + static_cast<uint64_t>(indices[j]), HETER ? values[j] : w_homo);
  }
}

inline unsigned grid_for(uint32_t items, uint32_t per_block) {
  const unsigned want = div_up(items, per_block);
  const unsigned cap = static_cast<unsigned>(device_info().num_cu) * 16u;
  return want < cap ? (want ? want : 1u) : cap;
}

// gpu_csr_event_sum_*: buffers = [events, indices, indptr, values, result]
template <typename F, typename I, bool HETER>
void csr_event_sum_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t len) {
  bpl_csr_event_sum_descriptor d;
  if (!unpack(target, opaque, len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  F *result = static_cast<F *>(buffers[4]);
  bool only_from_2_32 = false;
  if constexpr (sizeof(I) == 8) {
    // 64-bit index arrays and a result of more than 8,192 elements: the sorted event scatter reads them as they
    // are (a wave per active row and atomics in memory: 100,000 x 100,000 with 1e8 nonzeros at 5 % events 260 us)
    if (d.pre_size != 0 && d.post_size != 0) {
      const int done = csr_event_sum_wide<F, HETER>(target, stream, static_cast<const uint8_t *>(buffers[0]),
                                                    static_cast<const uint64_t *>(buffers[1]),
                                                    static_cast<const uint64_t *>(buffers[2]),
                                                    static_cast<const F *>(buffers[3]), result, d.pre_size, d.post_size);
      if (done < 0) return;
      only_from_2_32 = done > 0;
    }
  }
  if (!only_from_2_32) fill_zero(stream, result, d.post_size);
  if (d.pre_size == 0 || d.post_size == 0) return;
  hipLaunchKernelGGL((csr_event_sum_kernel<F, I, HETER>), dim3(grid_for(d.pre_size, kThreads / kWave)), dim3(kThreads),
                     0, stream, static_cast<const uint8_t *>(buffers[0]), static_cast<const I *>(buffers[1]),
                     static_cast<const I *>(buffers[2]), static_cast<const F *>(buffers[3]), result, d.pre_size,
                     only_from_2_32);
  check_launch(target);
}

// gpu_coo_event_sum_*: buffers = [events, pre_ids, post_ids, values, result]
template <typename F, typename I, bool HETER>
void coo_event_sum_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t len) {
  bpl_coo_sum_descriptor d;
  if (!unpack(target, opaque, len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  F *result = static_cast<F *>(buffers[4]);
  if (coo_window_sum<F, I, HETER, true>(target, stream, static_cast<const uint8_t *>(buffers[0]),
                                        static_cast<const F *>(buffers[3]), static_cast<const I *>(buffers[2]),
                                        static_cast<const I *>(buffers[1]), result, d.conn_size, d.post_size) != 0)
    return;  // (enqueued, or failed with its error standing)
  if (HETER && coo_bin_sum<F, I, true>(target, stream, static_cast<const uint8_t *>(buffers[0]),
                                       static_cast<const F *>(buffers[3]), static_cast<const I *>(buffers[2]),
                                       static_cast<const I *>(buffers[1]), result, d.conn_size, d.post_size) != 0)
    return;
  fill_zero(stream, result, d.post_size);
  if (d.conn_size == 0 || d.post_size == 0) return;
  hipLaunchKernelGGL((coo_event_sum_kernel<F, I, HETER>), dim3(grid_for(d.conn_size, kThreads)), dim3(kThreads), 0,
                     stream, static_cast<const uint8_t *>(buffers[0]), static_cast<const I *>(buffers[1]),
                     static_cast<const I *>(buffers[2]), static_cast<const F *>(buffers[3]), result, d.conn_size);
  check_launch(target);
}

// gpu_coo_atomic_sum_homo_*: buffers = [values, post_ids, result]
// gpu_coo_atomic_sum_heter_*: buffers = [values, post_ids, pre_ids, result]
template <typename F, typename I, bool HETER>
void coo_atomic_sum_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t len) {
  bpl_coo_sum_descriptor d;
  if (!unpack(target, opaque, len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  F *result = static_cast<F *>(buffers[HETER ? 3 : 2]);
  const I *post_ids = static_cast<const I *>(buffers[1]);
  const I *pre_ids = HETER ? static_cast<const I *>(buffers[2]) : post_ids;
  if (coo_window_sum<F, I, HETER, false>(target, stream, nullptr, static_cast<const F *>(buffers[0]), post_ids, pre_ids,
                                         result, d.conn_size, d.post_size) != 0)
    return;  // (enqueued, or failed with its error standing)
  if (HETER && coo_bin_sum<F, I, false>(target, stream, nullptr, static_cast<const F *>(buffers[0]), post_ids, pre_ids, result,
                                        d.conn_size, d.post_size) != 0)
    return;
  fill_zero(stream, result, d.post_size);
  if (d.conn_size == 0 || d.post_size == 0) return;
  hipLaunchKernelGGL((coo_atomic_sum_kernel<F, I, HETER>), dim3(grid_for(d.conn_size, kThreads)), dim3(kThreads), 0,
                     stream, static_cast<const F *>(buffers[0]), post_ids, pre_ids, result, d.conn_size);
  check_launch(target);
}

// gpu_coo_atomic_prod_homo_*: buffers = [values, post_ids, result]
// gpu_coo_atomic_prod_heter_*: buffers = [values, post_ids, pre_ids, result]
template <typename F, typename I, bool HETER>
void coo_atomic_prod_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t len) {
  bpl_coo_sum_descriptor d;
  if (!unpack(target, opaque, len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  F *result = static_cast<F *>(buffers[HETER ? 3 : 2]);
  if (d.post_size == 0) return;
  hipLaunchKernelGGL(fill_one_kernel<F>, dim3(div_up(d.post_size, kThreads)), dim3(kThreads), 0, stream, result,
                     d.post_size);
  if (d.conn_size != 0) {
    const I *post_ids = static_cast<const I *>(buffers[1]);
    const I *pre_ids = HETER ? static_cast<const I *>(buffers[2]) : post_ids;
    hipLaunchKernelGGL((coo_atomic_prod_kernel<F, I, HETER>), dim3(grid_for(d.conn_size, kThreads)), dim3(kThreads), 0,
                       stream, static_cast<const F *>(buffers[0]), post_ids, pre_ids, result, d.conn_size);
  }
  check_launch(target);
}

// gpu_csr_event_prod_*: buffers = [events, indices, indptr, values, result]
template <typename F, typename I, bool HETER>
void csr_event_prod_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t len) {
  bpl_csr_event_sum_descriptor d;
  if (!unpack(target, opaque, len, &d)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  F *result = static_cast<F *>(buffers[4]);
  if (d.post_size == 0) return;
  hipLaunchKernelGGL(fill_one_kernel<F>, dim3(div_up(d.post_size, kThreads)), dim3(kThreads), 0, stream, result,
                     d.post_size);
  if (d.pre_size != 0)
    hipLaunchKernelGGL((csr_event_prod_kernel<F, I, HETER>), dim3(grid_for(d.pre_size, kThreads / kWave)),
                       dim3(kThreads), 0, stream, static_cast<const uint8_t *>(buffers[0]),
                       static_cast<const I *>(buffers[1]), static_cast<const I *>(buffers[2]),
                       static_cast<const F *>(buffers[3]), result, d.pre_size);
  check_launch(target);
}

}  // namespace
}  // namespace bpl

#define BPL_DEFINE(name, call)                                                                   \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    hipStream_t s = static_cast<hipStream_t>(stream);                                            \
    using namespace bpl;                                                                         \
    call(__func__, s, buffers, opaque, opaque_len);                                              \
  }

BPL_DEFINE(gpu_csr_event_sum_homo_f32_i64, (csr_event_sum_entry<float, uint64_t, false>))
BPL_DEFINE(gpu_csr_event_sum_homo_f64_i64, (csr_event_sum_entry<double, uint64_t, false>))
BPL_DEFINE(gpu_csr_event_sum_heter_f32_i64, (csr_event_sum_entry<float, uint64_t, true>))
BPL_DEFINE(gpu_csr_event_sum_heter_f64_i64, (csr_event_sum_entry<double, uint64_t, true>))

BPL_DEFINE(gpu_coo_event_sum_homo_f32_i32, (coo_event_sum_entry<float, uint32_t, false>))
BPL_DEFINE(gpu_coo_event_sum_homo_f32_i64, (coo_event_sum_entry<float, uint64_t, false>))
BPL_DEFINE(gpu_coo_event_sum_homo_f64_i32, (coo_event_sum_entry<double, uint32_t, false>))
BPL_DEFINE(gpu_coo_event_sum_homo_f64_i64, (coo_event_sum_entry<double, uint64_t, false>))
BPL_DEFINE(gpu_coo_event_sum_heter_f32_i32, (coo_event_sum_entry<float, uint32_t, true>))
BPL_DEFINE(gpu_coo_event_sum_heter_f32_i64, (coo_event_sum_entry<float, uint64_t, true>))
BPL_DEFINE(gpu_coo_event_sum_heter_f64_i32, (coo_event_sum_entry<double, uint32_t, true>))
BPL_DEFINE(gpu_coo_event_sum_heter_f64_i64, (coo_event_sum_entry<double, uint64_t, true>))

BPL_DEFINE(gpu_coo_atomic_sum_homo_f32_i32, (coo_atomic_sum_entry<float, uint32_t, false>))
BPL_DEFINE(gpu_coo_atomic_sum_homo_f32_i64, (coo_atomic_sum_entry<float, uint64_t, false>))
BPL_DEFINE(gpu_coo_atomic_sum_homo_f64_i32, (coo_atomic_sum_entry<double, uint32_t, false>))
BPL_DEFINE(gpu_coo_atomic_sum_homo_f64_i64, (coo_atomic_sum_entry<double, uint64_t, false>))
BPL_DEFINE(gpu_coo_atomic_sum_heter_f32_i32, (coo_atomic_sum_entry<float, uint32_t, true>))
BPL_DEFINE(gpu_coo_atomic_sum_heter_f32_i64, (coo_atomic_sum_entry<float, uint64_t, true>))
BPL_DEFINE(gpu_coo_atomic_sum_heter_f64_i32, (coo_atomic_sum_entry<double, uint32_t, true>))
BPL_DEFINE(gpu_coo_atomic_sum_heter_f64_i64, (coo_atomic_sum_entry<double, uint64_t, true>))

BPL_DEFINE(gpu_coo_atomic_prod_homo_f32_i32, (coo_atomic_prod_entry<float, uint32_t, false>))
BPL_DEFINE(gpu_coo_atomic_prod_homo_f32_i64, (coo_atomic_prod_entry<float, uint64_t, false>))
BPL_DEFINE(gpu_coo_atomic_prod_homo_f64_i32, (coo_atomic_prod_entry<double, uint32_t, false>))
BPL_DEFINE(gpu_coo_atomic_prod_homo_f64_i64, (coo_atomic_prod_entry<double, uint64_t, false>))
BPL_DEFINE(gpu_coo_atomic_prod_heter_f32_i32, (coo_atomic_prod_entry<float, uint32_t, true>))
BPL_DEFINE(gpu_coo_atomic_prod_heter_f32_i64, (coo_atomic_prod_entry<float, uint64_t, true>))
BPL_DEFINE(gpu_coo_atomic_prod_heter_f64_i32, (coo_atomic_prod_entry<double, uint32_t, true>))
BPL_DEFINE(gpu_coo_atomic_prod_heter_f64_i64, (coo_atomic_prod_entry<double, uint64_t, true>))

BPL_DEFINE(gpu_csr_event_prod_homo_f32_i32, (csr_event_prod_entry<float, uint32_t, false>))
BPL_DEFINE(gpu_csr_event_prod_homo_f32_i64, (csr_event_prod_entry<float, uint64_t, false>))
BPL_DEFINE(gpu_csr_event_prod_homo_f64_i32, (csr_event_prod_entry<double, uint32_t, false>))
BPL_DEFINE(gpu_csr_event_prod_homo_f64_i64, (csr_event_prod_entry<double, uint64_t, false>))
BPL_DEFINE(gpu_csr_event_prod_heter_f32_i32, (csr_event_prod_entry<float, uint32_t, true>))
BPL_DEFINE(gpu_csr_event_prod_heter_f32_i64, (csr_event_prod_entry<float, uint64_t, true>))
BPL_DEFINE(gpu_csr_event_prod_heter_f64_i32, (csr_event_prod_entry<double, uint32_t, true>))
BPL_DEFINE(gpu_csr_event_prod_heter_f64_i64, (csr_event_prod_entry<double, uint64_t, true>))
