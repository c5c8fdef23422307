// Host-side runtime of libbrainpylib_amd.so: error channel, device properties, descriptor
// builders and the target registry.  Replaces the reference's lib/kernel_helpers.h,
// lib/kernel_helper_descriptor.cu and the Registrations() table of lib/gpu_ops.cc.
#include <atomic>
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
thread_local bool t_refused_by_capture = false;
// Set per device when a launch has failed: a pipeline that failed half way may have left the
// stream counters of that device nonzero (its last kernel, which resets them, never ran).
constexpr int kMaxDev = 64;
std::atomic<bool> g_counters_suspect[kMaxDev];
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
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev >= 0 && dev < kMaxDev) g_counters_suspect[dev].store(true);
    return false;
  }
  return true;
}

const DeviceInfo &device_info() {
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

namespace {
struct WorkspaceEntry {
  int dev;
  hipStream_t stream;
  void *ptr;
  size_t bytes;
};
std::vector<WorkspaceEntry> g_workspaces;
// Buffers that were handed out and then outgrown.  They stay allocated until the process ends:
// kernels enqueued earlier and HIP graphs captured earlier may still read and write them.
std::vector<WorkspaceEntry> g_retired;
std::mutex g_workspace_mu;

bool capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}
}  // namespace

bool scratch_refused_by_capture() { return t_refused_by_capture; }
void begin_call() { t_refused_by_capture = false; }
void ensure_error(const char *target, const char *why) {
  if (t_error.empty()) set_error("%s: %s", target, why);
}

void *stream_workspace(hipStream_t stream, size_t bytes) {
  t_refused_by_capture = false;
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lock(g_workspace_mu);
  WorkspaceEntry *e = nullptr;
  for (auto &x : g_workspaces)
    if (x.dev == dev && x.stream == stream) e = &x;
  if (e != nullptr && e->bytes >= bytes) return e->ptr;
  if (capturing(stream)) {
    set_error("scratch memory of %zu bytes is needed while the stream is being captured (it holds %zu): run the "
              "call once on this stream before capturing it", bytes, e ? e->bytes : size_t(0));
    t_refused_by_capture = true;
    return nullptr;
  }
  // A quarter of head room, and at least twice the buffer it replaces, so that the retired
  // buffers of a stream together stay below the size of its current one.
  size_t got = bytes + bytes / 4;
  if (e != nullptr && got < 2 * e->bytes) got = 2 * e->bytes;
  void *fresh = nullptr;
  if (hipMalloc(&fresh, got) != hipSuccess) {
    (void)hipGetLastError();
    fresh = nullptr;
    got = bytes;  // (once more without the head room)
    if (hipMalloc(&fresh, got) != hipSuccess) {
      (void)hipGetLastError();
      set_error("workspace allocation of %zu bytes failed", bytes);
      return nullptr;
    }
  }
  if (e == nullptr) {
    g_workspaces.push_back(WorkspaceEntry{dev, stream, nullptr, 0});
    e = &g_workspaces.back();
  }
  if (e->ptr != nullptr) g_retired.push_back(*e);
  e->ptr = fresh;
  e->bytes = got;
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
  t_refused_by_capture = false;
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lock(mu);
  if (dev >= 0 && dev < kMaxDev && g_counters_suspect[dev].exchange(false)) {
    // a launch failed on this device since the counters were last handed out: zero them all, each
    // on its own stream, before anything reads them again
    for (auto &x : entries)
      if (x.dev == dev) fill_zero(x.stream, x.ptr, static_cast<uint32_t>(kStreamCounterBytes / sizeof(uint32_t)));
  }
  for (auto &x : entries)
    if (x.dev == dev && x.stream == stream) return x.ptr;
  if (capturing(stream)) {
    set_error("the stream's counters would be allocated while it is being captured: run the call once on this "
              "stream before capturing it");
    t_refused_by_capture = true;
    return nullptr;
  }
  uint32_t *p = nullptr;
  if (hipMalloc(reinterpret_cast<void **>(&p), kStreamCounterBytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  // Zeroed by a kernel on the stream that will use them.  (hipMemset works on the null stream and does not
  // wait for the host; a non-blocking stream does not wait for the null stream either, so the first call on
  // such a stream could count its active rows before the zeros arrived and then lose the count to them.)
  fill_zero(stream, p, static_cast<uint32_t>(kStreamCounterBytes / sizeof(uint32_t)));
  entries.push_back(Entry{dev, stream, p});
  return p;
}

void *ScratchSource::request(size_t want, size_t need, size_t *got) const {
  if (need > want) want = need;
  if (!fixed()) {
    void *p = stream_workspace(stream, want);
    *got = p ? want : 0;
    if (p == nullptr && need < want && !t_refused_by_capture) {
      // the larger size could not be allocated: the least the caller can work with
      t_error.clear();
      p = stream_workspace(stream, need);
      *got = p ? need : 0;
    }
    return p;
  }
  if (need > arena_bytes) {
    set_error("the call needs %zu bytes of scratch memory and the allocation-free entry point holds %zu", need,
              arena_bytes);
    *got = 0;
    return nullptr;
  }
  *got = want < arena_bytes ? want : arena_bytes;
  return arena;
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

int bpl_stream_workspace_query(bpl_stream_t stream, void **ptr, size_t *bytes, size_t *retired_bytes) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lock(bpl::g_workspace_mu);
  void *p = nullptr;
  size_t n = 0, r = 0;
  for (const auto &x : bpl::g_workspaces)
    if (x.dev == dev && x.stream == static_cast<hipStream_t>(stream)) p = x.ptr, n = x.bytes;
  for (const auto &x : bpl::g_retired)
    if (x.dev == dev && x.stream == static_cast<hipStream_t>(stream)) r += x.bytes;
  if (ptr != nullptr) *ptr = p;
  if (bytes != nullptr) *bytes = n;
  if (retired_bytes != nullptr) *retired_bytes = r;
  return p != nullptr;
}

const char *bpl_last_error(void) { return bpl::t_error.c_str(); }
void bpl_clear_error(void) { bpl::t_error.clear(); }
const char *bpl_version(void) { return "0.1.0-gfx950"; }

}  // extern "C"
