/*
 * brainpylib_amd -- C ABI of the MI355X (gfx950) event-driven sparse operator library.
 *
 * Everything a host needs to drive the operators is declared here as plain `extern "C"`
 * symbols of libbrainpylib_amd.so: no C++ or framework types cross this boundary.
 *
 * The operator entry points are XLA GPU custom-call targets with the original 4-argument
 * ABI, and carry the same target NAMES the reference registers (the keys of its
 * `Registrations()` table, lib/gpu_ops.cc:24-177), so a host that looks targets up by name
 * finds them unchanged:
 *
 *     void target(hipStream_t stream, void **buffers, const char *opaque, size_t opaque_len);
 *
 *   stream      the HIP stream the call is enqueued on; the call returns without waiting.
 *   buffers     device pointers: all operands in the operator's order, then all results.
 *               Results may be uninitialised on entry; every element is written.
 *   opaque      byte image of one of the descriptor structs below (host memory, read before
 *               the call returns); opaque_len must equal sizeof(that struct).
 *
 * Errors never unwind through this boundary.  A call that fails validation or whose launch
 * fails enqueues nothing more, records a message retrievable with bpl_last_error() on the
 * calling thread and prints it to stderr.
 */
#ifndef BRAINPYLIB_AMD_H_
#define BRAINPYLIB_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* An opaque HIP stream handle (hipStream_t); declared as void* so that hosts without the HIP
 * headers can include this file. */
typedef void *bpl_stream_t;

typedef void (*bpl_target_fn)(bpl_stream_t stream, void **buffers, const char *opaque,
                              size_t opaque_len);

#define BPL_TARGET(name) \
  void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len)

/* ------------------------------------------------------------------------------------------
 * Descriptors (the `opaque` payloads).  Field order, types and padding are those of the
 * reference's structs, lib/kernel_helper_descriptor.cuh:42-144.
 * ---------------------------------------------------------------------------------------- */

/* lib/kernel_helper_descriptor.cuh:138-142 (TwoUintOneBoolDescriptor): event_csr_matvec. */
typedef struct {
  uint32_t n_row;    /* CSR shape[0] */
  uint32_t n_col;    /* CSR shape[1] */
  uint8_t transpose; /* C++ bool; 3 bytes of padding follow */
} bpl_twouint_onebool_descriptor;

/* Descriptor of the batched event_csr_matvec targets (no counterpart in the reference's GPU
 * library: brainpylib/_src/event_ops/event_csr_matvec.py:227-229 leaves the GPU translation of
 * `event_csr_matvec_batching_p` empty).  The fields are the static parameters and operand
 * shapes that the reference's CPU kernel reads, :152-193. */
typedef struct {
  uint32_t n_row;         /* CSR shape[0] */
  uint32_t n_col;         /* CSR shape[1] */
  uint32_t batch_size;    /* rows of the result */
  uint32_t values_batch;  /* leading dimension of every operand; entry bi uses row bi % dim */
  uint32_t indices_batch;
  uint32_t indptr_batch;
  uint32_t events_batch;
  uint32_t nnz;           /* second dimension of indices (and of values when heterogeneous) */
  uint8_t transpose;      /* 3 bytes of padding follow */
} bpl_event_csr_batching_descriptor;

/* lib/gpu_event_sum.cuh:10-13 (CSREventSumDescriptor): gpu_csr_event_sum_*. */
typedef struct {
  uint32_t pre_size;  /* rows of the CSR structure = length of events */
  uint32_t post_size; /* length of the result */
} bpl_csr_event_sum_descriptor;

/* lib/gpu_event_sum.cuh:38-41 (COOEventSumDescriptor) and lib/gpu_atomic_sum.cuh:10-13
 * (COOAtomicSumDescriptor): gpu_coo_event_sum_*, gpu_coo_atomic_sum_*. */
typedef struct {
  uint32_t conn_size; /* number of connections (length of post_ids) */
  uint32_t post_size; /* length of the result */
} bpl_coo_sum_descriptor;

/* lib/kernel_helper_descriptor.cuh:120-123 (DoubleSizeDescriptor): csr_matvec. */
typedef struct {
  uint32_t n_row;
  uint32_t n_col;
} bpl_double_size_descriptor;

/* Descriptor of the csr_matvec_transpose_* targets (own targets: the reference hands the
 * transposed product to cuSPARSE, brainpylib/_src/sparse_ops/cusparse_matvec.py:266-278).  The
 * 8-byte bpl_double_size_descriptor is accepted too; with the nonzero count the library can
 * size scratch memory for its sorted scatter of wide outputs. */
typedef struct {
  uint32_t n_row;
  uint32_t n_col;
  uint32_t nnz; /* length of indices = indptr[n_row] */
} bpl_csr_transpose_descriptor;

/* lib/kernel_helper_descriptor.cuh:42-45 (NonZeroDescriptor): event_info. */
typedef struct {
  uint32_t event_size;
  uint32_t batch_size;
} bpl_nonzero_descriptor;

/* lib/kernel_helper_descriptor.cuh:49-54 (JITConnProbHomoDescriptor).
 * n_row = number of outputs, n_col = number of inputs (already swapped for transpose=True);
 * log_p = log(1 - conn_prob), or log(1e-40) when conn_prob >= 1. */
typedef struct {
  uint32_t n_row;
  uint32_t n_col;
  uint32_t seed;
  double log_p;
} bpl_jitconn_prob_homo_descriptor;

/* lib/kernel_helper_descriptor.cuh:62-69 and :98-105 (JITConnProbUniformDescriptor /
 * JITConnProbNormalDescriptor; same layout).  uniform: w_a = w_min, w_b = w_range = w_high - w_low,
 * what the reference's GPU translation packs (brainpylib/_src/jitconn_ops/event_matvec.py:360-365);
 * a weight is canonical * w_range + w_min in the result type.  normal: w_a = w_mu, w_b = w_sigma. */
typedef struct {
  uint32_t n_row;
  uint32_t n_col;
  uint32_t seed;
  double log_p;
  double w_a;
  double w_b;
} bpl_jitconn_prob_weight_descriptor;

/* lib/kernel_helper_descriptor.cuh:80-88 (MatMatJITProbDescriptor1): Y[m,n] = X[m,k] @ M[k,n]. */
typedef struct {
  uint32_t m;
  uint32_t k;
  uint32_t n;
  uint32_t seed;
  double log_p;
  double w_a;
  double w_b;
} bpl_matmat_jit_prob_descriptor;

/* Builders: write the descriptor's byte image into `out` (capacity `cap`) and return its size,
 * or 0 if `cap` is too small.  They replace build_*_descriptor of
 * lib/kernel_helper_descriptor.cu:34-104.  Unlike the reference's builders, which narrow
 * log_p and the weight parameters to float before widening them again, these keep the
 * doubles, so the kernels see the same log_p as the reference's CPU path. */
size_t bpl_build_event_csr_batching_descriptor(uint32_t n_row, uint32_t n_col, uint32_t batch_size,
                                               uint32_t values_batch, uint32_t indices_batch,
                                               uint32_t indptr_batch, uint32_t events_batch, uint32_t nnz,
                                               int transpose, char *out, size_t cap);
/* lib/gpu_event_sum.cu:215-218,282-285, lib/gpu_atomic_sum.cu (build_*_descriptor) */
size_t bpl_build_csr_event_sum_descriptor(uint32_t pre_size, uint32_t post_size, char *out, size_t cap);
size_t bpl_build_coo_event_sum_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap);
size_t bpl_build_coo_atomic_sum_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap);
/* lib/gpu_atomic_prod.cu:104-107; brainpylib/_src/compat/event_prod.py:113 */
size_t bpl_build_coo_atomic_prod_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap);
size_t bpl_build_csr_event_prod_descriptor(uint32_t pre_size, uint32_t post_size, char *out, size_t cap);
size_t bpl_build_csr_transpose_descriptor(uint32_t n_row, uint32_t n_col, uint32_t nnz, char *out, size_t cap);
size_t bpl_build_twouint_onebool_descriptor(uint32_t n_row, uint32_t n_col, int transpose,
                                            char *out, size_t cap);
size_t bpl_build_double_size_descriptor(uint32_t n_row, uint32_t n_col, char *out, size_t cap);
size_t bpl_build_nonzero_descriptor(uint32_t event_size, uint32_t batch_size, char *out,
                                    size_t cap);
size_t bpl_build_jitconn_prob_homo_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed,
                                              double log_p, char *out, size_t cap);
size_t bpl_build_jitconn_prob_uniform_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed,
                                                 double log_p, double w_min, double w_range,
                                                 char *out, size_t cap);
size_t bpl_build_jitconn_prob_normal_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed,
                                                double log_p, double w_mu, double w_sigma,
                                                char *out, size_t cap);
size_t bpl_build_matmat_jit_prob_descriptor1(uint32_t m, uint32_t k, uint32_t n, uint32_t seed,
                                             double log_p, double w_a, double w_b, char *out,
                                             size_t cap);

/* ------------------------------------------------------------------------------------------
 * Registry: replaces Registrations() of lib/gpu_ops.cc:24-177.  Index i runs over
 * [0, bpl_num_targets()).
 * ---------------------------------------------------------------------------------------- */
int bpl_num_targets(void);
const char *bpl_target_name(int i);
bpl_target_fn bpl_target_function(int i);
bpl_target_fn bpl_find_target(const char *name); /* NULL if unknown */

/* Last error recorded on the calling thread ("" if none), and a reset. */
const char *bpl_last_error(void);
void bpl_clear_error(void);

/* Library version string. */
const char *bpl_version(void);

/* Scratch memory.  The custom-call ABI carries no workspace operand, so operators that need
 * staging memory (lists of active rows, sorted (column, weight) pairs, packed event bitmaps,
 * seeded generator states) take it from one allocation per (device, stream) that the library
 * makes with hipMalloc on first use and keeps until the process ends.  When a call needs more
 * than the stream's buffer holds, a larger buffer is allocated and the old one is retired but
 * never freed (earlier work and HIP graphs captured earlier may still use it).  While a stream is
 * being captured into a HIP graph nothing can be allocated: a call that would have to fails with
 * an error and enqueues nothing, so run every shape once on the stream before capturing it.
 * All graphs captured on one stream use that stream's buffer: their replays must be ordered with
 * each other and with eager calls on the capture stream (replaying two of them at once on
 * different streams, or one of them beside eager work on the capture stream, races on the buffer).
 * This query reports the current buffer of `stream` on the current device (its address and size)
 * and the bytes of retired buffers; it returns 0 if the stream has no buffer yet.  Any of the
 * three pointers may be NULL. */
int bpl_stream_workspace_query(bpl_stream_t stream, void **ptr, size_t *bytes, size_t *retired_bytes);

/* Self-check of the jitconn operators' skip computation (no counterpart in the reference, whose
 * kernels call log() per synapse, lib/gpu_jitconn_event_matvec.cu:94-110).  The kernels compute
 * ceil(log(U) / log_p) on a fast path (hardware fp32 log2) wherever the quotient is further from an
 * integer than a guard band, and as the CPU code does (lib/cpu_jitconn_event_matvec.cpp:24)
 * elsewhere.  This call evaluates both paths for n_draws values of U on the device: hashed ones, or
 * (near_boundaries != 0) values within 32 units in the last place of exp(k * log_p), k = 1, 2, ...
 * `counts` is device memory for four 64-bit words which the CALLER has zeroed: [0] += draws where
 * the fast path was trusted and differs from the exact one (must stay 0), [1] += draws inside the
 * guard band, [2] = max(old, bits of the largest |hardware log2(m) - log2(m)| over every fp32 m in
 * [0.5, 1) as a double), [3] = bits of the error of log2(U) that the guard band is built for, as a
 * double.  Returns 0 when the kernels were enqueued on `stream`. */
int bpl_selfcheck_jitconn_skips(bpl_stream_t stream, uint32_t seed, uint64_t n_draws, int near_boundaries,
                                double log_p, uint64_t *counts);

/* ------------------------------------------------------------------------------------------
 * event_csr_matvec  (lib/gpu_event_csr_matvec.cu:222-260; launchers :148-217)
 *   buffers = [data, indices, indptr, events, out]
 *     data     F[1] (homo) or F[nnz] (heter)
 *     indices  uint32/int32[nnz]        indptr  uint32/int32[n_row + 1]
 *     events   bool[.] (1 byte each) or F[.] (truthiness test); length n_row if transpose
 *              else n_col
 *     out      F[n_col] if transpose else F[n_row]
 *   opaque  = bpl_twouint_onebool_descriptor
 *   transpose:      out[indices[j]] += data[j]   for every j in row r, for every r with events[r]
 *   not transpose:  out[r] = sum of data[j] over j in row r with events[indices[j]]
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(event_csr_matvec_heter_float_bool);
BPL_TARGET(event_csr_matvec_heter_float_float);
BPL_TARGET(event_csr_matvec_heter_double_bool);
BPL_TARGET(event_csr_matvec_heter_double_double);
BPL_TARGET(event_csr_matvec_homo_float_bool);
BPL_TARGET(event_csr_matvec_homo_float_float);
BPL_TARGET(event_csr_matvec_homo_double_bool);
BPL_TARGET(event_csr_matvec_homo_double_double);

/* event_csr_matvec_heter_float_bool that allocates nothing.  No counterpart in the reference: it
 * is for callers that cannot allocate device memory inside the call -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same buffers, same descriptor,
 * same result as event_csr_matvec_heter_float_bool; the scratch memory that target takes from the
 * cached per-stream allocation (active-row list, counters, sorted runs, partial outputs, packed
 * bitmaps) lives in a static device array of 64 MiB (+ 256 bytes of counters) that every GPU
 * the library runs on holds until the process ends.  The call makes no hipMalloc / hipFree.
 *   Limits: a call whose scratch memory does not fit is rejected with an error and enqueues
 *   nothing.  transpose, more than 8,192 columns: 8 bytes per row + 128 KiB + 64 KiB per output
 *   window (at most 128 windows) must fit, i.e. any n_col with n_row <= 7,000,000; runs that
 *   overflow the rest of the array (about 7 million active nonzeros per call when n_row is
 *   100,000) are added with direct atomics, more slowly but correctly.  transpose, up to 8,192
 *   columns: 8 bytes per row.  no transpose: nothing up to 1,302,528 columns, n_col / 8 bytes +
 *   160 KiB beyond.
 *   All calls on one GPU share the array: calls that overlap on one GPU (different streams)
 *   race; calls on one stream, or ordered by events, are safe.
 *   May be captured cold: the first call of a process on a stream the library has never seen may
 *   be the captured one (the array's device address, kernel attributes and occupancy are looked
 *   up under the capture; none of these allocates).  The stream must belong to the current
 *   device. */
BPL_TARGET(event_csr_matvec_heter_float_bool_noalloc);

/* ------------------------------------------------------------------------------------------
 * event_csr_matvec_batching  (the batching rule's primitive,
 * brainpylib/_src/event_ops/event_csr_matvec.py:112-193, which the reference runs on the CPU
 * only; these targets have no counterpart in lib/gpu_ops.cc)
 *   buffers = [values, indices, indptr, events, out], row-major 2-D arrays:
 *     values   F[values_batch][1] or F[values_batch][nnz]
 *     indices  uint32/int32[indices_batch][nnz]   indptr  uint32/int32[indptr_batch][n_row + 1]
 *     events   bool or F [events_batch][n_row if transpose else n_col]
 *     out      F[batch_size][n_col if transpose else n_row]
 *   opaque  = bpl_event_csr_batching_descriptor
 *   out[bi] = event_csr_matvec(values[bi % values_batch], indices[bi % indices_batch],
 *                              indptr[bi % indptr_batch], events[bi % events_batch])
 *   With one shared matrix and transpose = 0 the column indices are streamed once per eight
 *   event vectors.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(event_csr_matvec_batching_heter_float_bool);
BPL_TARGET(event_csr_matvec_batching_heter_float_float);
BPL_TARGET(event_csr_matvec_batching_heter_double_bool);
BPL_TARGET(event_csr_matvec_batching_heter_double_double);
BPL_TARGET(event_csr_matvec_batching_homo_float_bool);
BPL_TARGET(event_csr_matvec_batching_homo_float_float);
BPL_TARGET(event_csr_matvec_batching_homo_double_bool);
BPL_TARGET(event_csr_matvec_batching_homo_double_double);

/* ------------------------------------------------------------------------------------------
 * The older operator family kept by brainpylib/_src/compat (lib/gpu_ops.cc:27-58).
 *   gpu_csr_event_sum_{homo,heter}_{f32,f64}_{i32,i64}  (lib/gpu_event_sum.cu:27-118,222-279)
 *     buffers = [events bool[pre_size], indices I[nnz], indptr I[pre_size + 1],
 *                values F[1] | F[nnz], result F[post_size]];  opaque = bpl_csr_event_sum_descriptor
 *     result[indices[j]] += values[j] for every j in row r, for every r with events[r]
 *   gpu_coo_event_sum_{homo,heter}_{f32,f64}_{i32,i64}  (lib/gpu_event_sum.cu:121-210,288-345)
 *     buffers = [events bool[.], pre_ids I[conn_size], post_ids I[conn_size],
 *                values F[1] | F[conn_size], result F[post_size]];  opaque = bpl_coo_sum_descriptor
 *     result[post_ids[i]] += values[i] for every connection i with events[pre_ids[i]]
 *   gpu_coo_atomic_sum_homo_{f32,f64}_{i32,i64}  (lib/gpu_atomic_sum.cu:27-60)
 *     buffers = [values F[1], post_ids I[conn_size], result F[post_size]]
 *   gpu_coo_atomic_sum_heter_{f32,f64}_{i32,i64}  (lib/gpu_atomic_sum.cu:62-98)
 *     buffers = [values F[.], post_ids I[conn_size], pre_ids I[conn_size], result F[post_size]]
 *     result[post_ids[i]] += values[pre_ids[i]];  opaque = bpl_coo_sum_descriptor
 *   I is a 32- or 64-bit integer read as unsigned.  The result is zeroed by the call.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_csr_event_sum_homo_f32_i32);
BPL_TARGET(gpu_csr_event_sum_homo_f32_i64);
BPL_TARGET(gpu_csr_event_sum_homo_f64_i32);
BPL_TARGET(gpu_csr_event_sum_homo_f64_i64);
BPL_TARGET(gpu_csr_event_sum_heter_f32_i32);
BPL_TARGET(gpu_csr_event_sum_heter_f32_i64);
BPL_TARGET(gpu_csr_event_sum_heter_f64_i32);
BPL_TARGET(gpu_csr_event_sum_heter_f64_i64);
BPL_TARGET(gpu_coo_event_sum_homo_f32_i32);
BPL_TARGET(gpu_coo_event_sum_homo_f32_i64);
BPL_TARGET(gpu_coo_event_sum_homo_f64_i32);
BPL_TARGET(gpu_coo_event_sum_homo_f64_i64);
BPL_TARGET(gpu_coo_event_sum_heter_f32_i32);
BPL_TARGET(gpu_coo_event_sum_heter_f32_i64);
BPL_TARGET(gpu_coo_event_sum_heter_f64_i32);
BPL_TARGET(gpu_coo_event_sum_heter_f64_i64);
BPL_TARGET(gpu_coo_atomic_sum_homo_f32_i32);
BPL_TARGET(gpu_coo_atomic_sum_homo_f32_i64);
BPL_TARGET(gpu_coo_atomic_sum_homo_f64_i32);
BPL_TARGET(gpu_coo_atomic_sum_homo_f64_i64);
BPL_TARGET(gpu_coo_atomic_sum_heter_f32_i32);
BPL_TARGET(gpu_coo_atomic_sum_heter_f32_i64);
BPL_TARGET(gpu_coo_atomic_sum_heter_f64_i32);
BPL_TARGET(gpu_coo_atomic_sum_heter_f64_i64);

/* The product twins: the result starts as ones and is multiplied, following the reference's CPU
 * kernels (lib/cpu_atomic_prod.cc:5-43, lib/cpu_event_prod.cc:5-55).
 *   gpu_coo_atomic_prod_homo_{f32,f64}_{i32,i64}   (registered at lib/gpu_ops.cc:60-64)
 *     buffers = [values F[1], post_ids I[conn_size], result F[post_size]]
 *   gpu_coo_atomic_prod_heter_{f32,f64}_{i32,i64}  (registered at lib/gpu_ops.cc:65-69)
 *     buffers = [values F[.], post_ids I[conn_size], pre_ids I[conn_size], result F[post_size]]
 *     result[post_ids[i]] *= values[pre_ids[i]];  opaque = bpl_coo_sum_descriptor
 *     (same layout as lib/gpu_atomic_prod.cuh:10-13; the reference's GPU kernels behind these
 *     names, lib/gpu_atomic_prod.cu:26-98, fill the result's bytes with 1 and add: not followed)
 *   gpu_csr_event_prod_{homo,heter}_{f32,f64}_{i32,i64}
 *     buffers = [events bool[pre_size], indices I[nnz], indptr I[pre_size + 1],
 *                values F[1] | F[nnz], result F[post_size]];  opaque = bpl_csr_event_sum_descriptor
 *     result[indices[j]] *= values[j] for every j in row r, for every r with events[r].
 *     The reference registers no such GPU target; these are the names its Python layer builds
 *     (brainpylib/_src/compat/event_prod.py:107-127, with build_csr_event_prod_descriptor(pre, post)).
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_coo_atomic_prod_homo_f32_i32);
BPL_TARGET(gpu_coo_atomic_prod_homo_f32_i64);
BPL_TARGET(gpu_coo_atomic_prod_homo_f64_i32);
BPL_TARGET(gpu_coo_atomic_prod_homo_f64_i64);
BPL_TARGET(gpu_coo_atomic_prod_heter_f32_i32);
BPL_TARGET(gpu_coo_atomic_prod_heter_f32_i64);
BPL_TARGET(gpu_coo_atomic_prod_heter_f64_i32);
BPL_TARGET(gpu_coo_atomic_prod_heter_f64_i64);
BPL_TARGET(gpu_csr_event_prod_homo_f32_i32);
BPL_TARGET(gpu_csr_event_prod_homo_f32_i64);
BPL_TARGET(gpu_csr_event_prod_homo_f64_i32);
BPL_TARGET(gpu_csr_event_prod_homo_f64_i64);
BPL_TARGET(gpu_csr_event_prod_heter_f32_i32);
BPL_TARGET(gpu_csr_event_prod_heter_f32_i64);
BPL_TARGET(gpu_csr_event_prod_heter_f64_i32);
BPL_TARGET(gpu_csr_event_prod_heter_f64_i64);

/* ------------------------------------------------------------------------------------------
 * csr_matvec  (lib/gpu_csr_matvec.cu:563-621; launchers :84-135,:195-246,:505-560)
 *   scalar / vector: buffers = [data, indices, indptr, vector, out]
 *   adaptive:        buffers = [data, indices, indptr, row_blocks, vector, out]
 *                    (row_blocks is accepted for layout compatibility and not read)
 *   opaque = bpl_double_size_descriptor;  out[r] = sum_j data[j] * vector[indices[j]], F[n_row].
 *   The three method names select the same kernel family here: the lanes-per-row mode is
 *   picked on the device from the mean row length.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(csr_matvec_heter_scalar_float);
BPL_TARGET(csr_matvec_heter_scalar_double);
BPL_TARGET(csr_matvec_heter_vector_float);
BPL_TARGET(csr_matvec_heter_vector_double);
BPL_TARGET(csr_matvec_heter_adaptive_float);
BPL_TARGET(csr_matvec_heter_adaptive_double);
BPL_TARGET(csr_matvec_homo_scalar_float);
BPL_TARGET(csr_matvec_homo_scalar_double);
BPL_TARGET(csr_matvec_homo_vector_float);
BPL_TARGET(csr_matvec_homo_vector_double);
BPL_TARGET(csr_matvec_homo_adaptive_float);
BPL_TARGET(csr_matvec_homo_adaptive_double);

/* Transposed csr_matvec: out[indices[j]] += vector[r] * data[j], out F[n_col].
 * The reference has no GPU kernel of its own for this orientation (it forwards to cuSPARSE,
 * brainpylib/_src/sparse_ops/cusparse_matvec.py:262-283); semantics follow its CPU loop
 * brainpylib/_src/sparse_ops/cusparse_matvec.py:195-212.
 *   buffers = [data, indices, indptr, vector(F[n_row]), out(F[n_col])],
 *   opaque = bpl_double_size_descriptor. */
BPL_TARGET(csr_matvec_transpose_heter_float);
BPL_TARGET(csr_matvec_transpose_heter_double);
BPL_TARGET(csr_matvec_transpose_homo_float);
BPL_TARGET(csr_matvec_transpose_homo_double);

/* ------------------------------------------------------------------------------------------
 * jitconn (event) matvec, version 2 kernels: y = M @ x with M regenerated on the fly.
 *   (lib/gpu_jitconn_event_matvec.cu:432-522, lib/gpu_jitconn_event_matvec_atomic.cu,
 *    lib/gpu_jitconn_matvec.cu:400-490, lib/gpu_jitconn_matvec_atomic.cu; names
 *    lib/gpu_ops.cc:107-158)
 *   buffers = [input, out]
 *     input  event targets: bool[n_col] (1 byte each) or F[n_col] (truthiness test)
 *            dense targets: F[n_col]
 *     out    F[n_row]
 *   opaque = bpl_jitconn_prob_homo_descriptor (homo) or bpl_jitconn_prob_weight_descriptor
 *            (uniform: w_a = low, w_b = high - low; normal: w_a = mean, w_b = stddev)
 *   Generator contract: stream i is std::mt19937{seed + i} with the libstdc++ distributions, walked
 *   exactly like the reference CPU kernels (lib/cpu_jitconn_event_matvec.cpp:20-31): output row i
 *   of a non-atomic target (input column i of an *_atomic_* target) equals what the reference CPU
 *   target computes for a matrix with that single stream and seed `seed + i`.  The reference's
 *   own backends disagree with each other on the matrix (one sequential mt19937 on CPU, cuRAND
 *   XORWOW per row on GPU); this library follows the CPU generator with the GPU's per-stream
 *   seeding.
 *   homo targets return counts (event input) or plain sums (dense input); the caller multiplies
 *   by the weight, as the reference does (brainpylib/_src/jitconn_ops/event_matvec.py:67-68).
 *   non-atomic ("outdim_parallel"): one stream per output row.  *_atomic_*: one stream per input
 *   column, accumulated with atomics.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_event_matvec_prob_homo_v2_float_bool);
BPL_TARGET(gpu_event_matvec_prob_homo_v2_float_float);
BPL_TARGET(gpu_event_matvec_prob_homo_v2_double_bool);
BPL_TARGET(gpu_event_matvec_prob_homo_v2_double_double);
BPL_TARGET(gpu_event_matvec_atomic_prob_homo_v2_float_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_homo_v2_float_float);
BPL_TARGET(gpu_event_matvec_atomic_prob_homo_v2_double_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_homo_v2_double_double);
BPL_TARGET(gpu_matvec_prob_homo_v2_float);
BPL_TARGET(gpu_matvec_prob_homo_v2_double);
BPL_TARGET(gpu_matvec_atomic_prob_homo_v2_float);
BPL_TARGET(gpu_matvec_atomic_prob_homo_v2_double);
BPL_TARGET(gpu_event_matvec_prob_uniform_v2_float_bool);
BPL_TARGET(gpu_event_matvec_prob_uniform_v2_float_float);
BPL_TARGET(gpu_event_matvec_prob_uniform_v2_double_bool);
BPL_TARGET(gpu_event_matvec_prob_uniform_v2_double_double);
BPL_TARGET(gpu_event_matvec_atomic_prob_uniform_v2_float_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_uniform_v2_float_float);
BPL_TARGET(gpu_event_matvec_atomic_prob_uniform_v2_double_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_uniform_v2_double_double);
BPL_TARGET(gpu_matvec_prob_uniform_v2_float);
BPL_TARGET(gpu_matvec_prob_uniform_v2_double);
BPL_TARGET(gpu_matvec_atomic_prob_uniform_v2_float);
BPL_TARGET(gpu_matvec_atomic_prob_uniform_v2_double);
BPL_TARGET(gpu_event_matvec_prob_normal_v2_float_bool);
BPL_TARGET(gpu_event_matvec_prob_normal_v2_float_float);
BPL_TARGET(gpu_event_matvec_prob_normal_v2_double_bool);
BPL_TARGET(gpu_event_matvec_prob_normal_v2_double_double);
BPL_TARGET(gpu_event_matvec_atomic_prob_normal_v2_float_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_normal_v2_float_float);
BPL_TARGET(gpu_event_matvec_atomic_prob_normal_v2_double_bool);
BPL_TARGET(gpu_event_matvec_atomic_prob_normal_v2_double_double);
BPL_TARGET(gpu_matvec_prob_normal_v2_float);
BPL_TARGET(gpu_matvec_prob_normal_v2_double);
BPL_TARGET(gpu_matvec_atomic_prob_normal_v2_float);
BPL_TARGET(gpu_matvec_atomic_prob_normal_v2_double);

/* ------------------------------------------------------------------------------------------
 * jitconn dense matvec under the reference's first-generation names (lib/gpu_ops.cc:143-148,
 * built by matvec.py:338-343,475-482,623-630 for version='v1', outdim_parallel=True only).
 *   buffers and descriptors as for the version 2 row walk, except that the descriptor's
 *   probability field holds conn_prob itself (lib/kernel_helper_descriptor.cuh:49-54); the
 *   library derives log_p = log(1 - conn_prob) (log(1e-40) at conn_prob >= 1) from it, as the
 *   reference's CPU path does for either version (matvec.py:296-308, one cpu_matvec_prob_* name
 *   for both).  The matrix therefore is the version 2 matrix: on the reference's CPU path the
 *   version does not change the result, and its own first-generation GPU kernels
 *   (a cuRAND Bernoulli test per entry, lib/gpu_jitconn_matvec.cu) are not followed.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_matvec_prob_homo_v1_float);
BPL_TARGET(gpu_matvec_prob_homo_v1_double);
BPL_TARGET(gpu_matvec_prob_uniform_v1_float);
BPL_TARGET(gpu_matvec_prob_uniform_v1_double);
BPL_TARGET(gpu_matvec_prob_normal_v1_float);
BPL_TARGET(gpu_matvec_prob_normal_v1_double);

/* ------------------------------------------------------------------------------------------
 * jitconn event matvec, first kernel generation ("hash" connectivity)
 *   (lib/gpu_jitconn_event_matvec.cu:10-79,138-215,281-362; names lib/gpu_ops.cc:107-112;
 *   generators lib/kernel_helpers_random.cuh:12-71)
 *   buffers = [event_ids (int32[n_col]: the positions of the events first, as nonzero_* lists
 *              them), event_num (int32[1]), out (F[n_row])]
 *   opaque = bpl_jitconn_prob_homo_descriptor (homo) or bpl_jitconn_prob_weight_descriptor
 *            (uniform: w_a = low, w_b = high - low; normal: w_a = mean, w_b = stddev), with the
 *            connection probability itself in the field `log_p` (the reference calls it `prob`)
 *   Synapse (row, col) exists iff lfsr113(seed + n_col * row + col) * 2^-32 < prob in 32-bit
 *   wrapping arithmetic (one step of LFSR113 from the state seed + {1, 7, 15, 127}); its weight
 *   is 1, taus88 * w_b + w_a, or w_a + sqrt(-2 log u) cos(2 pi v) * w_b with u, v the first two
 *   taus88 outputs from the state seed' + {1, 7, 15}.  out[row] adds the weights of the row's
 *   synapses to the listed columns, in list order.  A different matrix from the _v2 targets'.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_event_matvec_prob_homo_float);
BPL_TARGET(gpu_event_matvec_prob_homo_double);
BPL_TARGET(gpu_event_matvec_prob_uniform_float);
BPL_TARGET(gpu_event_matvec_prob_uniform_double);
BPL_TARGET(gpu_event_matvec_prob_normal_float);
BPL_TARGET(gpu_event_matvec_prob_normal_double);

/* ------------------------------------------------------------------------------------------
 * jitconn matmat: Y[m,n] = X[m,k] @ M[k,n], row-major X and Y, M regenerated on the fly
 *   (lib/gpu_jitconn_matmat.cu:279-317,364-455; names lib/gpu_ops.cc:161-174)
 *   buffers = [X (F[m*k]), Y (F[m*n])],  opaque = bpl_matmat_jit_prob_descriptor
 *   (normal: w_a = mean, w_b = stddev; uniform: w_a = low, w_b = high - low).
 *   Column j of M is generator stream seed + j over the k inputs, i.e. row i of Y equals the
 *   matvec target's result for X[i,:] with n_row = n, n_col = k (the reference tests' identity
 *   matmat == vmap(matvec(transpose=True)), brainpylib/_src/jitconn_ops/tests/matmat_testcase.py:133-138).
 *   The reference's experimental _v2/_v3 normal kernels generate a different matrix from _v1
 *   and from matvec and are not provided.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(gpu_matmat_prob_prob_normal_float_v1);
BPL_TARGET(gpu_matmat_prob_prob_normal_double_v1);
BPL_TARGET(gpu_matmat_prob_prob_uniform_float_v1);
BPL_TARGET(gpu_matmat_prob_prob_uniform_double_v1);

/* ------------------------------------------------------------------------------------------
 * event_info ("nonzero"): ordered positions of the nonzero events and their number
 *   (lib/gpu_event_info.cu:48-96; names lib/gpu_ops.cc:64-69)
 *   buffers = [events T[batch_size][event_size], event_ids int32[batch_size][event_size],
 *              event_num int32[batch_size]],  opaque = bpl_nonzero_descriptor
 *   event_ids rows: increasing positions, then -1 (the order of the reference's CPU kernel,
 *   brainpylib/_src/event_ops/event_info_collection.py:143-155; its GPU kernel leaves the order
 *   unspecified).  T = bool(1 byte) / int32 / int64 / float / double.  batch_size <= 65535.
 * ---------------------------------------------------------------------------------------- */
BPL_TARGET(nonzero_bool);
BPL_TARGET(nonzero_int);
BPL_TARGET(nonzero_long);
BPL_TARGET(nonzero_float);
BPL_TARGET(nonzero_double);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* BRAINPYLIB_AMD_H_ */
