// Sum of the windows that the workgroups of a scatter kernel left in scratch memory, shared by the
// kernels that finish such a scatter.
#pragma once
#include <cstdint>

#include <hip/hip_runtime.h>

namespace bpl {

// A workgroup of kSumCols * kSumSlices threads takes kSumCols columns; kSumSlices threads per column add every
// kSumSlices-th window, four loads in flight, and their sums are added in LDS in a fixed order (one thread per
// column through all the windows is a chain of hundreds of round trips).  partial: `groups` windows of n_col
// elements of type A; the sum is taken in S.  *mine: this thread holds the total of column
// blockIdx.x * kSumCols + threadIdx.x % kSumCols.
constexpr uint32_t kSumCols = 32, kSumSlices = 32;
template <typename S, typename A>
__device__ __forceinline__ S sum_windows_of_column(const A *__restrict__ partial, uint32_t n_col, uint32_t groups,
                                                   bool *mine) {
  __shared__ S s_part[kSumSlices][kSumCols + 1];
  const uint32_t lc = threadIdx.x % kSumCols, slice = threadIdx.x / kSumCols;
  const uint32_t c = blockIdx.x * kSumCols + lc;
  S acc = S(0);
  if (c < n_col) {
    const A *col = partial + c;
    uint32_t g = slice;
    for (; g + 3u * kSumSlices < groups; g += 4u * kSumSlices) {
      const A a0 = col[static_cast<size_t>(g) * n_col], a1 = col[static_cast<size_t>(g + kSumSlices) * n_col];
      const A a2 = col[static_cast<size_t>(g + 2u * kSumSlices) * n_col], a3 = col[static_cast<size_t>(g + 3u * kSumSlices) * n_col];
      acc = (((acc + a0) + a1) + a2) + a3;
    }
    for (; g < groups; g += kSumSlices) acc += col[static_cast<size_t>(g) * n_col];
  }
  s_part[slice][lc] = acc;
  __syncthreads();
  S total = S(0);
  *mine = slice == 0 && c < n_col;
  if (*mine) {
#pragma unroll
    for (uint32_t k = 0; k < kSumSlices; ++k) total += s_part[k][lc];
  }
  return total;
}

}  // namespace bpl
