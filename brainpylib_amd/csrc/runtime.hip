// Host-side runtime of libbrainpylib_amd.so: error channel, device properties, descriptor
// builders and the target registry.  Replaces the reference's lib/kernel_helpers.h,
// lib/kernel_helper_descriptor.cu and the Registrations() table of lib/gpu_ops.cc.
#include <cstdarg>
#include <cstddef>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "targets.h"

namespace bpl {

namespace {
thread_local std::string t_error;
}

void set_error(const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  t_error = buf;
  fprintf(stderr, "brainpylib_amd: %s\n", buf);
}

bool check_launch(const char *target) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", target, hipGetErrorString(e));
    return false;
  }
  return true;
}

const DeviceInfo &device_info() {
  constexpr int kMaxDev = 64;
  static DeviceInfo infos[kMaxDev];
  static bool known[kMaxDev] = {};
  static std::mutex mu;
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev < 0 || dev >= kMaxDev) dev = 0;
  std::lock_guard<std::mutex> lock(mu);
  if (!known[dev]) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      infos[dev].num_cu = prop.multiProcessorCount;
      infos[dev].lds_per_block = static_cast<int>(prop.sharedMemPerBlock);
    } else {
      infos[dev].num_cu = 256;
      infos[dev].lds_per_block = 64 * 1024;
    }
    known[dev] = true;
  }
  return infos[dev];
}

void *stream_workspace(hipStream_t stream, size_t bytes) {
  struct Entry {
    int dev;
    hipStream_t stream;
    void *ptr;
    size_t bytes;
  };
  static std::vector<Entry> entries;
  static std::mutex mu;
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lock(mu);
  Entry *e = nullptr;
  for (auto &x : entries)
    if (x.dev == dev && x.stream == stream) e = &x;
  if (e == nullptr) {
    entries.push_back(Entry{dev, stream, nullptr, 0});
    e = &entries.back();
  }
  if (e->bytes < bytes) {
    // the old buffer may still be read by work already enqueued on this stream
    if (e->ptr != nullptr) {
      (void)hipStreamSynchronize(stream);
      (void)hipFree(e->ptr);
      e->ptr = nullptr;
      e->bytes = 0;
    }
    const size_t want = bytes + bytes / 4;
    if (hipMalloc(&e->ptr, want) != hipSuccess) {
      (void)hipGetLastError();
      e->ptr = nullptr;
      set_error("workspace allocation of %zu bytes failed", want);
      return nullptr;
    }
    e->bytes = want;
  }
  return e->ptr;
}

uint32_t *stream_counters(hipStream_t stream) {
  struct Entry {
    int dev;
    hipStream_t stream;
    uint32_t *ptr;
  };
  static std::vector<Entry> entries;
  static std::mutex mu;
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lock(mu);
  for (auto &x : entries)
    if (x.dev == dev && x.stream == stream) return x.ptr;
  uint32_t *p = nullptr;
  constexpr size_t kBytes = 256;
  if (hipMalloc(reinterpret_cast<void **>(&p), kBytes) != hipSuccess || hipMemset(p, 0, kBytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  entries.push_back(Entry{dev, stream, p});
  return p;
}

}  // namespace bpl

// ---- layout checks against the reference's structs (lib/kernel_helper_descriptor.cuh) ----------
static_assert(sizeof(bpl_twouint_onebool_descriptor) == 12, "TwoUintOneBoolDescriptor is 12 bytes");
static_assert(offsetof(bpl_twouint_onebool_descriptor, transpose) == 8, "bool at offset 8");
static_assert(sizeof(bpl_event_csr_batching_descriptor) == 36, "batching descriptor is 36 bytes");
static_assert(sizeof(bpl_csr_event_sum_descriptor) == 8 && sizeof(bpl_coo_sum_descriptor) == 8,
              "CSREventSumDescriptor / COOEventSumDescriptor / COOAtomicSumDescriptor are 8 bytes");
static_assert(sizeof(bpl_double_size_descriptor) == 8, "DoubleSizeDescriptor is 8 bytes");
static_assert(sizeof(bpl_nonzero_descriptor) == 8, "NonZeroDescriptor is 8 bytes");
static_assert(sizeof(bpl_jitconn_prob_homo_descriptor) == 24, "JITConnProbHomoDescriptor is 24 bytes");
static_assert(offsetof(bpl_jitconn_prob_homo_descriptor, log_p) == 16, "double at offset 16");
static_assert(sizeof(bpl_jitconn_prob_weight_descriptor) == 40, "JITConnProb{Uniform,Normal}Descriptor is 40 bytes");
static_assert(offsetof(bpl_jitconn_prob_weight_descriptor, w_a) == 24, "w_a at offset 24");
static_assert(sizeof(bpl_matmat_jit_prob_descriptor) == 40, "MatMatJITProbDescriptor1 is 40 bytes");
static_assert(offsetof(bpl_matmat_jit_prob_descriptor, log_p) == 16, "log_p at offset 16");

namespace {
template <typename T>
size_t pack(const T &d, char *out, size_t cap) {
  if (out == nullptr || cap < sizeof(T)) return 0;
  std::memcpy(out, &d, sizeof(T));
  return sizeof(T);
}
}  // namespace

extern "C" {

size_t bpl_build_twouint_onebool_descriptor(uint32_t n_row, uint32_t n_col, int transpose, char *out,
                                            size_t cap) {
  bpl_twouint_onebool_descriptor d;
  std::memset(&d, 0, sizeof(d));
  d.n_row = n_row;
  d.n_col = n_col;
  d.transpose = transpose ? 1 : 0;
  return pack(d, out, cap);
}

size_t bpl_build_event_csr_batching_descriptor(uint32_t n_row, uint32_t n_col, uint32_t batch_size,
                                               uint32_t values_batch, uint32_t indices_batch,
                                               uint32_t indptr_batch, uint32_t events_batch, uint32_t nnz,
                                               int transpose, char *out, size_t cap) {
  bpl_event_csr_batching_descriptor d;
  std::memset(&d, 0, sizeof(d));
  d.n_row = n_row;
  d.n_col = n_col;
  d.batch_size = batch_size;
  d.values_batch = values_batch;
  d.indices_batch = indices_batch;
  d.indptr_batch = indptr_batch;
  d.events_batch = events_batch;
  d.nnz = nnz;
  d.transpose = transpose ? 1 : 0;
  return pack(d, out, cap);
}

size_t bpl_build_csr_event_sum_descriptor(uint32_t pre_size, uint32_t post_size, char *out, size_t cap) {
  bpl_csr_event_sum_descriptor d{pre_size, post_size};
  return pack(d, out, cap);
}

size_t bpl_build_coo_event_sum_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap) {
  bpl_coo_sum_descriptor d{conn_size, post_size};
  return pack(d, out, cap);
}

size_t bpl_build_coo_atomic_sum_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap) {
  bpl_coo_sum_descriptor d{conn_size, post_size};
  return pack(d, out, cap);
}

size_t bpl_build_coo_atomic_prod_descriptor(uint32_t conn_size, uint32_t post_size, char *out, size_t cap) {
  bpl_coo_sum_descriptor d{conn_size, post_size};
  return pack(d, out, cap);
}

size_t bpl_build_csr_event_prod_descriptor(uint32_t pre_size, uint32_t post_size, char *out, size_t cap) {
  bpl_csr_event_sum_descriptor d{pre_size, post_size};
  return pack(d, out, cap);
}

size_t bpl_build_csr_transpose_descriptor(uint32_t n_row, uint32_t n_col, uint32_t nnz, char *out, size_t cap) {
  bpl_csr_transpose_descriptor d{n_row, n_col, nnz};
  return pack(d, out, cap);
}

size_t bpl_build_double_size_descriptor(uint32_t n_row, uint32_t n_col, char *out, size_t cap) {
  bpl_double_size_descriptor d{n_row, n_col};
  return pack(d, out, cap);
}

size_t bpl_build_nonzero_descriptor(uint32_t event_size, uint32_t batch_size, char *out, size_t cap) {
  bpl_nonzero_descriptor d{event_size, batch_size};
  return pack(d, out, cap);
}

size_t bpl_build_jitconn_prob_homo_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed, double log_p,
                                              char *out, size_t cap) {
  bpl_jitconn_prob_homo_descriptor d;
  std::memset(&d, 0, sizeof(d));
  d.n_row = n_row;
  d.n_col = n_col;
  d.seed = seed;
  d.log_p = log_p;
  return pack(d, out, cap);
}

static size_t build_weight(uint32_t n_row, uint32_t n_col, uint32_t seed, double log_p, double a, double b,
                           char *out, size_t cap) {
  bpl_jitconn_prob_weight_descriptor d;
  std::memset(&d, 0, sizeof(d));
  d.n_row = n_row;
  d.n_col = n_col;
  d.seed = seed;
  d.log_p = log_p;
  d.w_a = a;
  d.w_b = b;
  return pack(d, out, cap);
}

size_t bpl_build_jitconn_prob_uniform_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed, double log_p,
                                                 double w_min, double w_range, char *out, size_t cap) {
  return build_weight(n_row, n_col, seed, log_p, w_min, w_range, out, cap);
}

size_t bpl_build_jitconn_prob_normal_descriptor(uint32_t n_row, uint32_t n_col, uint32_t seed, double log_p,
                                                double w_mu, double w_sigma, char *out, size_t cap) {
  return build_weight(n_row, n_col, seed, log_p, w_mu, w_sigma, out, cap);
}

size_t bpl_build_matmat_jit_prob_descriptor1(uint32_t m, uint32_t k, uint32_t n, uint32_t seed, double log_p,
                                             double w_a, double w_b, char *out, size_t cap) {
  bpl_matmat_jit_prob_descriptor d;
  std::memset(&d, 0, sizeof(d));
  d.m = m;
  d.k = k;
  d.n = n;
  d.seed = seed;
  d.log_p = log_p;
  d.w_a = w_a;
  d.w_b = w_b;
  return pack(d, out, cap);
}

// ---- registry --------------------------------------------------------------------------------
namespace {
struct Entry {
  const char *name;
  bpl_target_fn fn;
};
#define BPL_X(name) {#name, &name},
const Entry kTargets[] = {BPL_ALL_TARGETS(BPL_X)};
#undef BPL_X
constexpr int kNumTargets = static_cast<int>(sizeof(kTargets) / sizeof(kTargets[0]));
}  // namespace

int bpl_num_targets(void) { return kNumTargets; }
const char *bpl_target_name(int i) { return (i >= 0 && i < kNumTargets) ? kTargets[i].name : nullptr; }
bpl_target_fn bpl_target_function(int i) { return (i >= 0 && i < kNumTargets) ? kTargets[i].fn : nullptr; }
bpl_target_fn bpl_find_target(const char *name) {
  if (name == nullptr) return nullptr;
  for (int i = 0; i < kNumTargets; ++i)
    if (std::strcmp(kTargets[i].name, name) == 0) return kTargets[i].fn;
  return nullptr;
}

const char *bpl_last_error(void) { return bpl::t_error.c_str(); }
void bpl_clear_error(void) { bpl::t_error.clear(); }
const char *bpl_version(void) { return "0.1.0-gfx950"; }

}  // extern "C"
