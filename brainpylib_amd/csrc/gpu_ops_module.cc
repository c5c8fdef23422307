// Python module `brainpylib_amd.gpu_ops`: the interface the reference's Python layer expects
// from its `gpu_ops` extension (lib/gpu_ops.cc:179-198): `registrations()` returning
// {target name: PyCapsule("xla._CUSTOM_CALL_TARGET")} and `build_*_descriptor(...)` returning
// the opaque bytes.  It is a thin wrapper over the C ABI of libbrainpylib_amd.so and contains no
// device code.
#include <pybind11/pybind11.h>

#include <string>

#include "../../include/brainpylib_amd.h"

namespace py = pybind11;

namespace {

py::dict Registrations() {
  py::dict dict;
  const int n = bpl_num_targets();
  for (int i = 0; i < n; ++i)
    dict[bpl_target_name(i)] =
        py::capsule(reinterpret_cast<void *>(bpl_target_function(i)), "xla._CUSTOM_CALL_TARGET");
  return dict;
}

// Calls a C-ABI builder with a stack buffer appended to its arguments.
#define BPL_PACK(fn, ...)                                              \
  [&]() {                                                              \
    char bpl_buf_[64];                                                 \
    const size_t bpl_len_ = fn(__VA_ARGS__, bpl_buf_, sizeof(bpl_buf_)); \
    if (bpl_len_ == 0) throw std::runtime_error("descriptor does not fit"); \
    return py::bytes(std::string(bpl_buf_, bpl_len_));                 \
  }()

}  // namespace

PYBIND11_MODULE(gpu_ops, m) {
  m.doc() = "XLA custom-call targets and descriptor builders of brainpylib_amd (gfx950)";
  m.def("registrations", &Registrations);
  m.def("build_event_csr_batching_descriptor",
        [](uint32_t n_row, uint32_t n_col, uint32_t batch_size, uint32_t values_batch, uint32_t indices_batch,
           uint32_t indptr_batch, uint32_t events_batch, uint32_t nnz, bool transpose) {
          return BPL_PACK(bpl_build_event_csr_batching_descriptor, n_row, n_col, batch_size, values_batch,
                          indices_batch, indptr_batch, events_batch, nnz, transpose ? 1 : 0);
        });
  m.def("build_csr_event_sum_descriptor",
        [](uint32_t pre_size, uint32_t post_size) { return BPL_PACK(bpl_build_csr_event_sum_descriptor, pre_size, post_size); });
  m.def("build_coo_event_sum_descriptor",
        [](uint32_t conn_size, uint32_t post_size) { return BPL_PACK(bpl_build_coo_event_sum_descriptor, conn_size, post_size); });
  m.def("build_coo_atomic_sum_descriptor",
        [](uint32_t conn_size, uint32_t post_size) { return BPL_PACK(bpl_build_coo_atomic_sum_descriptor, conn_size, post_size); });
  m.def("build_coo_atomic_prod_descriptor",
        [](uint32_t conn_size, uint32_t post_size) { return BPL_PACK(bpl_build_coo_atomic_prod_descriptor, conn_size, post_size); });
  m.def("build_csr_event_prod_descriptor",
        [](uint32_t pre_size, uint32_t post_size) { return BPL_PACK(bpl_build_csr_event_prod_descriptor, pre_size, post_size); });
  m.def("build_csr_transpose_descriptor", [](uint32_t n_row, uint32_t n_col, uint32_t nnz) {
    return BPL_PACK(bpl_build_csr_transpose_descriptor, n_row, n_col, nnz);
  });
  m.def("build_twouint_onebool_descriptor", [](uint32_t x, uint32_t y, bool b) {
    return BPL_PACK(bpl_build_twouint_onebool_descriptor, x, y, b ? 1 : 0);
  });
  m.def("build_double_size_descriptor",
        [](uint32_t x, uint32_t y) { return BPL_PACK(bpl_build_double_size_descriptor, x, y); });
  m.def("build_nonzero_descriptor", [](uint32_t event_size, uint32_t batch_size) {
    return BPL_PACK(bpl_build_nonzero_descriptor, event_size, batch_size);
  });
  // prob / weights are taken as double (Python floats): the reference narrows them to float
  m.def("build_jitconn_prob_homo_descriptor", [](uint32_t n_row, uint32_t n_col, uint32_t seed, double prob) {
    return BPL_PACK(bpl_build_jitconn_prob_homo_descriptor, n_row, n_col, seed, prob);
  });
  m.def("build_jitconn_prob_uniform_descriptor",
        [](uint32_t n_row, uint32_t n_col, uint32_t seed, double prob, double w_min, double w_range) {
          return BPL_PACK(bpl_build_jitconn_prob_uniform_descriptor, n_row, n_col, seed, prob, w_min, w_range);
        });
  m.def("build_jitconn_prob_normal_descriptor",
        [](uint32_t n_row, uint32_t n_col, uint32_t seed, double prob, double w_mu, double w_sigma) {
          return BPL_PACK(bpl_build_jitconn_prob_normal_descriptor, n_row, n_col, seed, prob, w_mu, w_sigma);
        });
  m.def("build_matmat_jit_prob_descriptor1",
        [](uint32_t mm, uint32_t k, uint32_t n, uint32_t seed, double log_p, double w1, double w2) {
          return BPL_PACK(bpl_build_matmat_jit_prob_descriptor1, mm, k, n, seed, log_p, w1, w2);
        });
}
