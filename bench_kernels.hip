// Measurement kernels of bench.py (gfx950): the ceilings that the operators' rooflines are set
// beside, measured on the device the benchmark runs on.  Not part of libbrainpylib_amd.so.
//
//   bench_gather_fma   acc += x[idx[j]] * w[j] over a flat index / weight stream, no row structure:
//                      what csr_matvec does per nonzero (two coalesced streams and one random
//                      4-byte read of the vector), at the same occupancy.  Its rate is the ceiling
//                      of any CSR product that gathers the vector from L2.
//   bench_stream       plain 16-byte loads over a buffer, at the same occupancy: the HBM read
//                      rate a streaming kernel reaches on this device.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

template <int U>
__global__ __launch_bounds__(1024) void gather_fma_kernel(const float *__restrict__ x, const uint32_t *__restrict__ idx,
                                                          const float *__restrict__ w, float *__restrict__ out,
                                                          uint64_t n) {
  const uint64_t total = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t gtid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  double acc = 0.0;
  uint64_t base = gtid;
  for (; base + (U - 1) * total < n; base += U * total) {
    uint32_t c[U];
    float d[U];
#pragma unroll
    for (int u = 0; u < U; ++u) c[u] = idx[base + u * total], d[u] = w[base + u * total];
#pragma unroll
    for (int u = 0; u < U; ++u) acc += static_cast<double>(x[c[u]] * d[u]);
  }
  for (; base < n; base += total) acc += static_cast<double>(x[idx[base]] * w[base]);
  out[gtid] = static_cast<float>(acc);
}

__global__ __launch_bounds__(1024) void stream_kernel(const uint4 *__restrict__ p, uint32_t *__restrict__ out,
                                                      uint64_t n16) {
  constexpr int U = 4;
  const uint64_t total = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t gtid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  uint64_t base = gtid;
  for (; base + (U - 1) * total < n16; base += U * total) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = p[base + u * total];
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; base < n16; base += total) {
    const uint4 v = p[base];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  out[gtid] = acc;
}

}  // namespace

extern "C" {

// out: blocks * threads floats.  loads_in_flight: 2, 4 or 8 gathers per lane.  Returns 0 on success.
int bench_gather_fma(void *stream, const float *x, const uint32_t *idx, const float *w, float *out, uint64_t n,
                     int blocks, int threads, int loads_in_flight) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (blocks <= 0 || threads <= 0 || threads > 1024) return 1;
  if (loads_in_flight == 2) hipLaunchKernelGGL(gather_fma_kernel<2>, dim3(blocks), dim3(threads), 0, s, x, idx, w, out, n);
  else if (loads_in_flight == 4) hipLaunchKernelGGL(gather_fma_kernel<4>, dim3(blocks), dim3(threads), 0, s, x, idx, w, out, n);
  else if (loads_in_flight == 8) hipLaunchKernelGGL(gather_fma_kernel<8>, dim3(blocks), dim3(threads), 0, s, x, idx, w, out, n);
  else return 1;
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// p: n16 16-byte words; out: blocks * threads words.
int bench_stream(void *stream, const void *p, void *out, uint64_t n16, int blocks, int threads) {
  if (blocks <= 0 || threads <= 0 || threads > 1024) return 1;
  hipLaunchKernelGGL(stream_kernel, dim3(blocks), dim3(threads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4 *>(p), static_cast<uint32_t *>(out), n16);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // extern "C"
