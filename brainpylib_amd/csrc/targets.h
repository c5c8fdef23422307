// X-macro list of every custom-call target exported by libbrainpylib_amd.so.  It must name
// exactly the BPL_TARGET declarations of include/brainpylib_amd.h (a CPU test compares them).
#pragma once

#define BPL_EVENT_CSR_TARGETS(X)            \
  X(event_csr_matvec_heter_float_bool)      \
  X(event_csr_matvec_heter_float_float)     \
  X(event_csr_matvec_heter_double_bool)     \
  X(event_csr_matvec_heter_double_double)   \
  X(event_csr_matvec_homo_float_bool)       \
  X(event_csr_matvec_homo_float_float)      \
  X(event_csr_matvec_homo_double_bool)      \
  X(event_csr_matvec_homo_double_double)    \
  X(event_csr_matvec_heter_float_bool_noalloc)

#define BPL_CSR_TARGETS(X)                  \
  X(csr_matvec_heter_scalar_float)          \
  X(csr_matvec_heter_scalar_double)         \
  X(csr_matvec_heter_vector_float)          \
  X(csr_matvec_heter_vector_double)         \
  X(csr_matvec_heter_adaptive_float)        \
  X(csr_matvec_heter_adaptive_double)       \
  X(csr_matvec_homo_scalar_float)           \
  X(csr_matvec_homo_scalar_double)          \
  X(csr_matvec_homo_vector_float)           \
  X(csr_matvec_homo_vector_double)          \
  X(csr_matvec_homo_adaptive_float)         \
  X(csr_matvec_homo_adaptive_double)        \
  X(csr_matvec_transpose_heter_float)       \
  X(csr_matvec_transpose_heter_double)      \
  X(csr_matvec_transpose_homo_float)        \
  X(csr_matvec_transpose_homo_double)

#define BPL_JITCONN_TARGETS(X) \
  X(gpu_event_matvec_prob_homo_v2_float_bool) \
  X(gpu_event_matvec_prob_homo_v2_float_float) \
  X(gpu_event_matvec_prob_homo_v2_double_bool) \
  X(gpu_event_matvec_prob_homo_v2_double_double) \
  X(gpu_event_matvec_atomic_prob_homo_v2_float_bool) \
  X(gpu_event_matvec_atomic_prob_homo_v2_float_float) \
  X(gpu_event_matvec_atomic_prob_homo_v2_double_bool) \
  X(gpu_event_matvec_atomic_prob_homo_v2_double_double) \
  X(gpu_matvec_prob_homo_v2_float) \
  X(gpu_matvec_prob_homo_v2_double) \
  X(gpu_matvec_atomic_prob_homo_v2_float) \
  X(gpu_matvec_atomic_prob_homo_v2_double) \
  X(gpu_event_matvec_prob_uniform_v2_float_bool) \
  X(gpu_event_matvec_prob_uniform_v2_float_float) \
  X(gpu_event_matvec_prob_uniform_v2_double_bool) \
  X(gpu_event_matvec_prob_uniform_v2_double_double) \
  X(gpu_event_matvec_atomic_prob_uniform_v2_float_bool) \
  X(gpu_event_matvec_atomic_prob_uniform_v2_float_float) \
  X(gpu_event_matvec_atomic_prob_uniform_v2_double_bool) \
  X(gpu_event_matvec_atomic_prob_uniform_v2_double_double) \
  X(gpu_matvec_prob_uniform_v2_float) \
  X(gpu_matvec_prob_uniform_v2_double) \
  X(gpu_matvec_atomic_prob_uniform_v2_float) \
  X(gpu_matvec_atomic_prob_uniform_v2_double) \
  X(gpu_event_matvec_prob_normal_v2_float_bool) \
  X(gpu_event_matvec_prob_normal_v2_float_float) \
  X(gpu_event_matvec_prob_normal_v2_double_bool) \
  X(gpu_event_matvec_prob_normal_v2_double_double) \
  X(gpu_event_matvec_atomic_prob_normal_v2_float_bool) \
  X(gpu_event_matvec_atomic_prob_normal_v2_float_float) \
  X(gpu_event_matvec_atomic_prob_normal_v2_double_bool) \
  X(gpu_event_matvec_atomic_prob_normal_v2_double_double) \
  X(gpu_matvec_prob_normal_v2_float) \
  X(gpu_matvec_prob_normal_v2_double) \
  X(gpu_matvec_atomic_prob_normal_v2_float) \
  X(gpu_matvec_atomic_prob_normal_v2_double) \
  X(gpu_matvec_prob_homo_v1_float) \
  X(gpu_matvec_prob_homo_v1_double) \
  X(gpu_matvec_prob_uniform_v1_float) \
  X(gpu_matvec_prob_uniform_v1_double) \
  X(gpu_matvec_prob_normal_v1_float) \
  X(gpu_matvec_prob_normal_v1_double)

#define BPL_JITCONN_HASH_TARGETS(X) \
  X(gpu_event_matvec_prob_homo_float) \
  X(gpu_event_matvec_prob_homo_double) \
  X(gpu_event_matvec_prob_uniform_float) \
  X(gpu_event_matvec_prob_uniform_double) \
  X(gpu_event_matvec_prob_normal_float) \
  X(gpu_event_matvec_prob_normal_double)

#define BPL_MATMAT_TARGETS(X) \
  X(gpu_matmat_prob_prob_normal_float_v1) \
  X(gpu_matmat_prob_prob_normal_double_v1) \
  X(gpu_matmat_prob_prob_uniform_float_v1) \
  X(gpu_matmat_prob_prob_uniform_double_v1)

#define BPL_NONZERO_TARGETS(X) \
  X(nonzero_bool) \
  X(nonzero_int) \
  X(nonzero_long) \
  X(nonzero_float) \
  X(nonzero_double)

#define BPL_EVENT_CSR_BATCHING_TARGETS(X)            \
  X(event_csr_matvec_batching_heter_float_bool)      \
  X(event_csr_matvec_batching_heter_float_float)     \
  X(event_csr_matvec_batching_heter_double_bool)     \
  X(event_csr_matvec_batching_heter_double_double)   \
  X(event_csr_matvec_batching_homo_float_bool)       \
  X(event_csr_matvec_batching_homo_float_float)      \
  X(event_csr_matvec_batching_homo_double_bool)      \
  X(event_csr_matvec_batching_homo_double_double)

#define BPL_COMPAT_TARGETS(X) \
  X(gpu_csr_event_sum_homo_f32_i32) \
  X(gpu_csr_event_sum_homo_f32_i64) \
  X(gpu_csr_event_sum_homo_f64_i32) \
  X(gpu_csr_event_sum_homo_f64_i64) \
  X(gpu_csr_event_sum_heter_f32_i32) \
  X(gpu_csr_event_sum_heter_f32_i64) \
  X(gpu_csr_event_sum_heter_f64_i32) \
  X(gpu_csr_event_sum_heter_f64_i64) \
  X(gpu_coo_event_sum_homo_f32_i32) \
  X(gpu_coo_event_sum_homo_f32_i64) \
  X(gpu_coo_event_sum_homo_f64_i32) \
  X(gpu_coo_event_sum_homo_f64_i64) \
  X(gpu_coo_event_sum_heter_f32_i32) \
  X(gpu_coo_event_sum_heter_f32_i64) \
  X(gpu_coo_event_sum_heter_f64_i32) \
  X(gpu_coo_event_sum_heter_f64_i64) \
  X(gpu_coo_atomic_sum_homo_f32_i32) \
  X(gpu_coo_atomic_sum_homo_f32_i64) \
  X(gpu_coo_atomic_sum_homo_f64_i32) \
  X(gpu_coo_atomic_sum_homo_f64_i64) \
  X(gpu_coo_atomic_sum_heter_f32_i32) \
  X(gpu_coo_atomic_sum_heter_f32_i64) \
  X(gpu_coo_atomic_sum_heter_f64_i32) \
  X(gpu_coo_atomic_sum_heter_f64_i64) \
  X(gpu_coo_atomic_prod_homo_f32_i32) \
  X(gpu_coo_atomic_prod_homo_f32_i64) \
  X(gpu_coo_atomic_prod_homo_f64_i32) \
  X(gpu_coo_atomic_prod_homo_f64_i64) \
  X(gpu_coo_atomic_prod_heter_f32_i32) \
  X(gpu_coo_atomic_prod_heter_f32_i64) \
  X(gpu_coo_atomic_prod_heter_f64_i32) \
  X(gpu_coo_atomic_prod_heter_f64_i64) \
  X(gpu_csr_event_prod_homo_f32_i32) \
  X(gpu_csr_event_prod_homo_f32_i64) \
  X(gpu_csr_event_prod_homo_f64_i32) \
  X(gpu_csr_event_prod_homo_f64_i64) \
  X(gpu_csr_event_prod_heter_f32_i32) \
  X(gpu_csr_event_prod_heter_f32_i64) \
  X(gpu_csr_event_prod_heter_f64_i32) \
  X(gpu_csr_event_prod_heter_f64_i64)

#define BPL_ALL_TARGETS(X)  \
  BPL_EVENT_CSR_TARGETS(X)  \
  BPL_EVENT_CSR_BATCHING_TARGETS(X) \
  BPL_CSR_TARGETS(X)        \
  BPL_JITCONN_TARGETS(X)    \
  BPL_JITCONN_HASH_TARGETS(X) \
  BPL_MATMAT_TARGETS(X)     \
  BPL_NONZERO_TARGETS(X)    \
  BPL_COMPAT_TARGETS(X)
