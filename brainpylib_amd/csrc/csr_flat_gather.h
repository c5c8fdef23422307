// csr_matvec without transpose for vectors that are gathered from L2 (csr_flat_gather.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace bpl {

// The flat walk computes positions of nonzeros one step beyond the end of a wave's range in 32 bits: matrices
// with more nonzeros than this are left to the caller's other kernel, whatever their mean.
constexpr uint32_t kFlatMaxNnz = 0xffffffffu - 8192u;

// y = A x, walked flat: every wave owns a contiguous range of the nonzeros and tells the rows apart through
// windows of indptr in LDS.  For matrices with min_mean <= nnz / n_row < max_mean and nnz <= kFlatMaxNnz; for others the kernels
// return at once and write nothing (the mean is known on the device only, so the caller enqueues its kernel
// for short rows behind this one).  x must have at least one element.  Takes 20 bytes of the stream's scratch
// memory per wave of its launch.
enum class FlatGather { kEnqueued, kNotApplicable /* an array is not 16-byte aligned: nothing done, no error */,
                        kFailed /* no scratch memory, or the launch failed: error recorded */ };
template <typename F>
FlatGather csr_flat_gather(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                     const uint32_t *indptr, const F *x, F *y, uint32_t n_row, uint32_t min_mean, uint32_t max_mean);

}  // namespace bpl
