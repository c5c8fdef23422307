// csr_matvec without transpose for vectors that are gathered from L2 (csr_quad_gather.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace bpl {

// y = A x over rows of at least `min_mean` nonzeros on average; with a shorter mean the kernel returns at
// once and writes nothing (the mean is known on the device only, so the caller enqueues its kernel for
// short rows behind this one).  x must have at least one element.  False if nothing was enqueued (the
// index or weight array is not 16-byte aligned) or the launch failed (error recorded).
template <typename F>
bool csr_quad_gather(const char *target, hipStream_t stream, const F *data, bool heter, const uint32_t *indices,
                     const uint32_t *indptr, const F *x, F *y, uint32_t n_row, uint32_t min_mean);

}  // namespace bpl
