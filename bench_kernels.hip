// Measurement kernels of bench.py (gfx950): the ceilings that the operators' rooflines are set
// beside, measured on the device the benchmark runs on.  Not part of libbrainpylib_amd.so.
//
//   bench_gather_fma   acc += x[idx[j]] * w[j] over a flat index / weight stream, no row structure:
//                      what csr_matvec does per nonzero (two coalesced streams and one random
//                      4-byte read of the vector), at the same occupancy.  Its rate is the ceiling
//                      of any CSR product that gathers the vector from L2.
//   bench_gather_fma4  the same with the two streams read 16 bytes per lane (four consecutive nonzeros per
//                      request), optionally with the nontemporal hint, and with the lanes of an
//                      instruction reading either one contiguous kilobyte or eight pieces of 128 bytes
//                      (what groups of 8 lanes per CSR row read).
//   bench_stream       plain 16-byte loads over a buffer, at the same occupancy: the HBM read
//                      rate a streaming kernel reaches on this device.
//   bench_lds_atomic   random read-modify-writes into a 64 KB LDS window from 1,024-thread workgroups:
//                      ds_add_f32, ds_add_u32, ds_add_f64, plain LDS writes, or the address arithmetic
//                      alone (to subtract).  The rates the choice of accumulator types rests on.
//   bench_global_atomic  fp32 atomic adds to random elements of a vector in device memory, and 32-bit
//                      integer adds that all go to ONE address (one lane per workgroup): what a
//                      scatter through atomics and a shared fill counter cost per operation.
//   bench_l2_read      16-byte loads over a buffer small enough to stay in every L2, read again and
//                      again: the rate at which the L2s deliver lines to the compute units.
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

// A wave takes blocks of U * 64 consecutive quads.  SEG lanes read consecutive quads in one instruction:
// SEG = 64: an instruction reads 1 KB in one piece; SEG = 8: it reads 8 pieces of 128 bytes that lie
// U * 128 bytes apart.
template <int U, bool NT, int SEG>
__global__ __launch_bounds__(1024) void gather_fma4_kernel(const float *__restrict__ x, const uint4 *__restrict__ idx,
                                                           const float4 *__restrict__ w, float *__restrict__ out,
                                                           uint64_t n4) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const uint32_t lane = threadIdx.x % 64;
  const uint64_t waves = static_cast<uint64_t>(gridDim.x) * (blockDim.x / 64);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64;
  double acc = 0.0;
  for (uint64_t b = wave; (b + 1) * (U * 64) <= n4; b += waves) {
    u32x4 c[U];
    f32x4 d[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t at = b * (U * 64) + (lane / SEG) * (U * SEG) + u * SEG + lane % SEG;
      if (NT) {
        c[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(idx) + at);
        d[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(w) + at);
      } else {
        c[u] = reinterpret_cast<const u32x4 *>(idx)[at];
        d[u] = reinterpret_cast<const f32x4 *>(w)[at];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float a0 = x[c[u].x] * d[u].x, a1 = x[c[u].y] * d[u].y, a2 = x[c[u].z] * d[u].z, a3 = x[c[u].w] * d[u].w;
      acc += static_cast<double>(a0);
      acc += static_cast<double>(a1);
      acc += static_cast<double>(a2);
      acc += static_cast<double>(a3);
    }
  }
  // the quads that do not fill a block
  const uint64_t done = n4 / (U * 64) * (U * 64);
  for (uint64_t at = done + wave * 64 + lane; at < n4; at += waves * 64) {
    const uint4 c = idx[at];
    const float4 d = w[at];
    acc += static_cast<double>(x[c.x] * d.x);
    acc += static_cast<double>(x[c.y] * d.y);
    acc += static_cast<double>(x[c.z] * d.z);
    acc += static_cast<double>(x[c.w] * d.w);
  }
  out[static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x] = static_cast<float>(acc);
}

typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));
template <bool NT>
__device__ __forceinline__ stream_u32x4 stream_word(const stream_u32x4 *p) {
  return NT ? __builtin_nontemporal_load(p) : *p;
}
// NT: the loads are marked nontemporal, as the kernels mark the arrays they read once.
template <bool NT>
__global__ __launch_bounds__(1024) void stream_kernel(const stream_u32x4 *__restrict__ p, uint32_t *__restrict__ out,
                                                      uint64_t n16) {
  constexpr int U = 4;
  const uint64_t total = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t gtid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  uint64_t base = gtid;
  for (; base + (U - 1) * total < n16; base += U * total) {
    stream_u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = stream_word<NT>(p + base + u * total);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; base < n16; base += total) {
    const stream_u32x4 v = stream_word<NT>(p + base);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  out[gtid] = acc;
}

__device__ __forceinline__ uint32_t lcg_step(uint32_t &s) {
  s = s * 1664525u + 1013904223u;
  return s >> 8;
}

// MODE 0: ds_add_f32   1: ds_add_u32   2: ds_add_f64   3: ds_write_b32   4: the addresses only
template <int MODE>
__global__ __launch_bounds__(1024) void lds_atomic_kernel(float *__restrict__ out, int iters) {
  __shared__ float win[16384];  // 64 KB
  for (int i = threadIdx.x; i < 16384; i += 1024) win[i] = 0.f;
  __syncthreads();
  uint32_t st = (blockIdx.x * 1024u + threadIdx.x) * 2654435761u + 12345u;
  float acc = 0.f;
  for (int i = 0; i < iters; ++i) {
    const uint32_t a = lcg_step(st) & 16383u;
    if (MODE == 0) atomicAdd(&win[a], 1.0f);
    else if (MODE == 1) atomicAdd(reinterpret_cast<uint32_t *>(&win[a]), 1u);
    else if (MODE == 2) atomicAdd(reinterpret_cast<double *>(&win[a & 16382u]), 1.0);
    else if (MODE == 3) win[a] = 1.0f;
    else acc += static_cast<float>(a);
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = win[5] + acc;
}

// Returning 32-bit additions in LDS where G neighbouring lanes share a counter (a wave's counters differ from
// the other waves'); every addition depends on the answer of the one before it.
template <int G>
__global__ __launch_bounds__(1024) void lds_shared_counter_kernel(float *__restrict__ out, int iters) {
  __shared__ uint32_t cnt[4096];
  for (int i = threadIdx.x; i < 4096; i += 1024) cnt[i] = 0u;
  __syncthreads();
  const uint32_t lane = threadIdx.x % 64u, wave = threadIdx.x / 64u;
  uint32_t acc = 0;
  for (int i = 0; i < iters; ++i) acc += atomicAdd(&cnt[(wave * 64u + lane / G + (acc & 1u)) & 4095u], 1u);
  out[blockIdx.x] = static_cast<float>(__builtin_amdgcn_readfirstlane(static_cast<int>(acc)) & 1);
}

// fp32 atomic adds (no return value) to random elements of y[0, n)
__global__ __launch_bounds__(256) void global_atomic_random_kernel(float *__restrict__ y, uint32_t n, int iters) {
  uint32_t st = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
  for (int i = 0; i < iters; ++i) unsafeAtomicAdd(&y[lcg_step(st) % n], 1.0f);
}

// one lane per workgroup adds `iters` times to ONE counter (no return value)
__global__ __launch_bounds__(64) void global_atomic_same_address_kernel(uint32_t *__restrict__ counter, int iters) {
  if (threadIdx.x == 0)
    for (int i = 0; i < iters; ++i) atomicAdd(counter, 1u);
}

__global__ __launch_bounds__(1024) void l2_read_kernel(const uint4 *__restrict__ p, uint32_t *__restrict__ out,
                                                       uint32_t n16, int repeats) {
  // every workgroup reads the whole buffer `repeats` times, beginning at a place of its own
  uint32_t acc = 0;
  const uint32_t begin = (blockIdx.x * 4099u) % n16;
  for (int r = 0; r < repeats; ++r) {
    for (uint32_t i = threadIdx.x; i < n16; i += 4 * 1024) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        uint32_t at = begin + i + u * 1024u;
        at = at >= n16 ? at - n16 : at;
        at = at >= n16 ? at - n16 : at;
        v[u] = p[at];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
  }
  out[blockIdx.x * 1024u + threadIdx.x] = acc;
}

}  // namespace

extern "C" {

// out: blocks floats.  mode 0: ds_add_f32, 1: ds_add_u32, 2: ds_add_f64, 3: ds_write_b32, 4: addresses only;
// 101, 104, 116: returning 32-bit additions with 1, 4, 16 neighbouring lanes per counter.
// blocks * 1024 * iters operations per launch.
int bench_lds_atomic(void *stream, float *out, int blocks, int iters, int mode) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (blocks <= 0 || iters <= 0) return 1;
  if (mode == 0) hipLaunchKernelGGL(lds_atomic_kernel<0>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 1) hipLaunchKernelGGL(lds_atomic_kernel<1>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 2) hipLaunchKernelGGL(lds_atomic_kernel<2>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 3) hipLaunchKernelGGL(lds_atomic_kernel<3>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 4) hipLaunchKernelGGL(lds_atomic_kernel<4>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 101) hipLaunchKernelGGL(lds_shared_counter_kernel<1>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 104) hipLaunchKernelGGL(lds_shared_counter_kernel<4>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else if (mode == 116) hipLaunchKernelGGL(lds_shared_counter_kernel<16>, dim3(blocks), dim3(1024), 0, s, out, iters);
  else return 1;
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// same_address == 0: blocks * 256 * iters fp32 adds to random elements of y[0, n) (y: n floats).
// same_address != 0: blocks * iters integer adds to the first word of y, one lane per workgroup.
int bench_global_atomic(void *stream, void *y, uint32_t n, int blocks, int iters, int same_address) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (blocks <= 0 || iters <= 0 || n == 0) return 1;
  if (same_address)
    hipLaunchKernelGGL(global_atomic_same_address_kernel, dim3(blocks), dim3(64), 0, s, static_cast<uint32_t *>(y), iters);
  else
    hipLaunchKernelGGL(global_atomic_random_kernel, dim3(blocks), dim3(256), 0, s, static_cast<float *>(y), n, iters);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// p: n16 16-byte words (a multiple of 4,096, small enough for the L2); out: blocks * 1,024 words.
// blocks * repeats * n16 * 16 bytes are read per launch.
int bench_l2_read(void *stream, const void *p, void *out, uint32_t n16, int repeats, int blocks) {
  if (blocks <= 0 || repeats <= 0 || n16 == 0 || n16 % 4096 != 0) return 1;
  hipLaunchKernelGGL(l2_read_kernel, dim3(blocks), dim3(1024), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4 *>(p), static_cast<uint32_t *>(out), n16, repeats);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

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

// The same over n (a multiple of 4) nonzeros with 16-byte stream loads.  quads_in_flight 1, 2 or 4;
// nontemporal != 0: the two streams are read with the nontemporal hint; pieces: 1 or 8 (see the kernel).
int bench_gather_fma4(void *stream, const float *x, const uint32_t *idx, const float *w, float *out, uint64_t n,
                      int blocks, int threads, int quads_in_flight, int nontemporal, int pieces) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (blocks <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0 || n % 4 != 0) return 1;
  if (pieces != 1 && pieces != 8) return 1;
  const uint4 *i4 = reinterpret_cast<const uint4 *>(idx);
  const float4 *w4 = reinterpret_cast<const float4 *>(w);
#define BPL_LAUNCH4(U, NT, SEG) \
  hipLaunchKernelGGL((gather_fma4_kernel<U, NT, SEG>), dim3(blocks), dim3(threads), 0, s, x, i4, w4, out, n / 4)
#define BPL_PICK(U)                                   \
  do {                                                \
    if (nontemporal && pieces == 1) BPL_LAUNCH4(U, true, 64);  \
    else if (nontemporal) BPL_LAUNCH4(U, true, 8);    \
    else if (pieces == 1) BPL_LAUNCH4(U, false, 64);  \
    else BPL_LAUNCH4(U, false, 8);                    \
  } while (0)
  if (quads_in_flight == 1) BPL_PICK(1);
  else if (quads_in_flight == 2) BPL_PICK(2);
  else if (quads_in_flight == 4) BPL_PICK(4);
  else return 1;
#undef BPL_PICK
#undef BPL_LAUNCH4
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// p: n16 16-byte words; out: blocks * threads words.
int bench_stream(void *stream, const void *p, void *out, uint64_t n16, int blocks, int threads, int nontemporal) {
  if (blocks <= 0 || threads <= 0 || threads > 1024) return 1;
  auto kernel = nontemporal ? stream_kernel<true> : stream_kernel<false>;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const stream_u32x4 *>(p), static_cast<uint32_t *>(out), n16);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // extern "C"
