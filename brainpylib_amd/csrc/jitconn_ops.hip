// Just-in-time-connectivity operators for gfx950: the matrix is never stored, its rows are
// regenerated in registers on every call from per-stream std::mt19937 generators (mt_wave.h)
// with geometric skip sampling, exactly the loop of the reference's CPU kernels
//   first = ceil(log(U)/log_p);  while (i < n) { [w = weight draw;] use(i, w); i += ceil(log(U)/log_p); }
// (lib/cpu_jitconn_event_matvec.cpp:20-31, lib/cpu_jitconn_matvec.cpp:20-29 and their *_atomic
// twins).  Stream `o` is std::mt19937{seed + o}.
//
// One wave64 owns one stream.  Each lane draws one synapse of the next batch (its skip and its
// weight), a DPP prefix sum over the skips places the 64 synapses, a ballot finds where the row
// ends.  The only memory traffic is the input vector (events are packed into an LDS bitmap when
// it fits) and the output.
//
//   row walk  ("outdim_parallel"):  stream per output element, inputs gathered, one store.
//   column walk ("atomic"):         stream per input element, silent inputs are skipped
//                                   entirely (compacted per workgroup), outputs by atomics.
//
// Reference boundary: lib/gpu_jitconn_event_matvec.cu:111-135,432-522,
// lib/gpu_jitconn_event_matvec_atomic.cu:61-85, lib/gpu_jitconn_matvec.cu:115-138,
// lib/gpu_jitconn_matvec_atomic.cu:53-77 (buffers = [input, out]; descriptors; target names).
#include <cmath>

#include <type_traits>

#include "bins.h"
#include "common.h"
#include "jitconn_stream.h"
#include "targets.h"

namespace bpl {
namespace {

// ---- row walk -------------------------------------------------------------------------------------
// LDS the row walk gives to an event bitmap when it wants two 16-wave workgroups per CU (each wave
// can issue one instruction every four cycles, so the number of resident waves bounds the VALU
// utilisation: 32 waves per CU walk 290 G synapses/s, the 15 that fit beside a 125 KB bitmap 228).
constexpr uint32_t kRowwalkCoarseBytes = 38912;

// BITS: where the event probes go.  0: the event vector in global memory; 1: its bitmap in LDS;
// 2: a coarse bitmap in LDS (one bit per 2^g inputs, at most kRowwalkCoarseBytes) and, where its
// bit is set, the exact packed bitmap in global memory (`in`, the coarse one behind it).
// (With the coarse bitmap two 16-wave workgroups are meant to share a CU: 8 waves per SIMD, which
// the register allocation has to leave room for; the normal-weight walk needs 66 otherwise.)
// Register budget: eight waves per SIMD need at most 64 vector AND at most 80 scalar registers per
// wave here (with 81..96 scalar registers only seven fit, so a second 16-wave workgroup does not).
constexpr uint32_t kFuseBatch = 64;   // streams seeded together, one per lane
constexpr uint32_t kFuseSlots = 3;    // batches of seeded states in a workgroup's ring
constexpr uint32_t kFuseSpin = 1u << 22;           // polls of a flag in LDS before a wave stops waiting
constexpr uint32_t kFuseNotSeeded = 0x80000000u;   // flag bit: the batch's rows seed their own generators
constexpr size_t kFuseRingBytes = static_cast<size_t>(kFuseSlots) * kFuseBatch * kMtN * sizeof(uint32_t);  // per workgroup
static_assert(kMtSeedTileWords <= kMtStateWords, "the seeding wave transposes through its own state buffer");

template <typename T1, typename VT, int IN, int W, int BITS, bool FUSED>
__global__ __launch_bounds__(1024, (BITS == 2 || (W == kNormal && sizeof(T1) == 4)) ? 8 : 4)
    __attribute__((amdgpu_num_sgpr(80))) void jitconn_rowwalk_kernel(const VT *__restrict__ in, T1 *__restrict__ out,
                                                               uint32_t n_out, uint32_t n_in, uint32_t seed,
                                                               double log_p, T1 wa, T1 wb, uint32_t first,
                                                               uint32_t *states) {
  // Handles the n_out outputs first .. first + n_out - 1; `states` (optional) holds their
  // generators' seeded states.  FUSED: all outputs from 0, `states` is the workgroups' rings
  // (kFuseRingBytes each).
  extern __shared__ __attribute__((aligned(8))) uint32_t smem[];
  const int lane = lane_id();
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t nwaves = blockDim.x / kWave;
  constexpr int kWords = StreamLds<T1, W>::words;
  uint32_t *st = smem + wave * kWords;
  const uint32_t *bits = smem + nwaves * kWords;
  uint32_t coarse_g = 0, coarse_g5 = 5;
  if constexpr (BITS == 2) {
    uint32_t *wbits = smem + nwaves * kWords;
    coarse_g = coarse_shift(n_in, kRowwalkCoarseBytes);
    coarse_g5 = coarse_g + 5u;
    const uint32_t words = (coarse_bits(n_in, coarse_g) + 31u) >> 5;
    const uint32_t *coarse = reinterpret_cast<const uint32_t *>(in) + coarse_offset_words(n_in);
    for (uint32_t i = threadIdx.x; i < words; i += blockDim.x) wbits[i] = coarse[i];
    __syncthreads();
  } else if constexpr (BITS == 1) {
    uint32_t *wbits = smem + nwaves * kWords;
    const uint32_t words = (n_in + 31u) >> 5;
    for (uint32_t i = threadIdx.x; i < words; i += blockDim.x) wbits[i] = pack_events32<VT>(in, i << 5, n_in);
    __syncthreads();
  }
  // output o from stream seed + o, whose seeded state is at `pre` (or nullptr: the wave seeds it itself)
  auto walk_row = [&](uint32_t o, const uint32_t *pre, auto &&loaded) {
    double acc = 0.0;
    uint32_t cnt = 0;
    // two-level bitmap: the exact word of a batch is requested when the batch is drawn and looked
    // at when the next one is, so that no wave waits for it
    uint32_t late_word = 0, late_idx = 0;
    uint64_t late_coarse = 0;  // lanes whose coarse bit was set (wave uniform, so the scalar unit combines the masks)
    bool late_lane = false;    // this lane's bit of it
    T1 late_w = T1(0);
    auto settle = [&]() {
      const bool bit = __builtin_amdgcn_ubfe(late_word, late_idx, 1u) != 0u;
      if (W == kHomo) cnt += static_cast<uint32_t>(__popcll(late_coarse & __builtin_amdgcn_ballot_w64(bit)));
      else if (bit && late_lane) acc += static_cast<double>(late_w);
    };
    walk_stream<T1, W>(st, lane, seed + o, pre, n_in, log_p, wa, wb, [&](uint32_t idx, T1 w, bool valid) {
      if constexpr (IN == kInEvent && BITS == 2) {
        settle();
        // bit c = idx >> g of the coarse bitmap: word c >> 5, bit c & 31 (the bit-field extract takes the
        // low five bits).  Lanes past the end of the row extract a field of width 0, which is 0 whatever
        // the word holds: the word they read may lie past the bitmap, even past the workgroup's LDS
        // (such a read returns 0 and cannot fault), and its value is never looked at.
        const uint32_t c = idx >> coarse_g;
        const bool coarse = __builtin_amdgcn_ubfe(bits[idx >> coarse_g5], c, valid ? 1u : 0u) != 0u;
        // (lanes without a coarse hit read word 0 and ignore it: a plain load for the whole wave)
        late_word = reinterpret_cast<const uint32_t *>(in)[coarse ? idx >> 5 : 0u];
        late_idx = idx;
        late_coarse = __builtin_amdgcn_ballot_w64(coarse);
        late_lane = coarse;
        late_w = w;
        return;
      }
      if (IN == kInDense) {
        if (valid) {
          const T1 v = static_cast<T1>(in[idx]);
          acc += static_cast<double>(W == kHomo ? v : static_cast<T1>(w * v));
        }
      } else {
        bool hit = false;
        if (valid) {
          if (BITS == 1) hit = (bits[idx >> 5] >> (idx & 31u)) & 1u;
          else hit = probe_event(in, idx);
        }
        if (W == kHomo) cnt += static_cast<uint32_t>(__popcll(__ballot(hit)));
        else if (hit) acc += static_cast<double>(w);
      }
    }, loaded);
    if constexpr (IN == kInEvent && BITS == 2) settle();
    if (IN == kInEvent && W == kHomo) {
      if (lane == 0) out[o] = static_cast<T1>(cnt);
    } else {
      acc = wave_sum(acc);
      if (lane == 0) out[o] = static_cast<T1>(acc);
    }
  };

  if constexpr (!FUSED) {
    for (uint32_t i = blockIdx.x * nwaves + wave; i < n_out; i += gridDim.x * nwaves)
      walk_row(first + i, states ? states + static_cast<size_t>(i) * kMtN : nullptr, NoLoadHook());
  } else {
    // The generators are seeded inside the kernel, 64 streams at a time on the vector unit (the scalar
    // unit, one per CU, cannot seed a stream per wave fast enough), while the other waves walk: the
    // workgroup takes batches of 64 consecutive outputs (batch blockIdx.x + j * gridDim.x is its j-th),
    // its waves take (batch, row) tasks from a counter in LDS, and the wave that takes the first row of
    // batch j first seeds batch j + 1 into slot (j + 1) % 3 of the workgroup's ring of seeded states in
    // device memory (`states`), which stays in the L2.  A slot is written again only after all 64 rows
    // of its previous batch have copied their state to LDS, and read only after its flag says which
    // batch it holds; every wait is bounded, and a wave that gives up seeds its own generator instead.
    __shared__ uint32_t s_task, s_ready[kFuseSlots], s_loaded[kFuseSlots];
    const uint32_t n_batches = (n_out + kFuseBatch - 1u) / kFuseBatch;
    const uint32_t mine = n_batches > blockIdx.x ? (n_batches - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;
    // (`states` is neither const nor restrict: other waves write what this one reads behind a flag)
    uint32_t *ring = states + static_cast<size_t>(blockIdx.x) * kFuseSlots * kFuseBatch * kMtN;
    if (threadIdx.x == 0) {
      s_task = 0;
      for (uint32_t k = 0; k < kFuseSlots; ++k) s_ready[k] = 0, s_loaded[k] = 0;
    }
    __syncthreads();
    if (mine == 0) return;
    auto seed_batch = [&](uint32_t j) {
      const uint32_t slot = j % kFuseSlots;
      mt_seed_batch(st, lane, seed + (blockIdx.x + j * gridDim.x) * kFuseBatch + static_cast<uint32_t>(lane),
                    ring + static_cast<size_t>(slot) * kFuseBatch * kMtN);
      __hip_atomic_store(&s_ready[slot], j + 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    if (wave == 0) seed_batch(0);
    for (;;) {
      // Every lane adds one, so the counter advances by 64 per task and any lane's old value / 64 is the
      // task.  (With the add under `if (lane == 0)` the compiler split the loop by lane: lane 0 went back
      // to the add alone and the other lanes stayed behind with task 0 for ever.)
      const uint32_t t = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(
                             static_cast<int>(atomicAdd(&s_task, 1u)))) / kWave;
      const uint32_t j = t / kFuseBatch, r = t % kFuseBatch;
      if (j >= mine) break;
      if (r == 0 && j + 1 < mine) {
        // slot (j + 1) % 3 last held batch j - 2: (j + 1) / 3 batches have used it, 64 loads each
        const uint32_t slot = (j + 1u) % kFuseSlots, need = ((j + 1u) / kFuseSlots) * kFuseBatch;
        bool free_ = false;
        for (uint32_t spin = 0; spin < kFuseSpin && !free_; ++spin) {
          free_ = __hip_atomic_load(&s_loaded[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= need;
          if (!free_) __builtin_amdgcn_s_sleep(2);
        }
        if (free_) seed_batch(j + 1u);
        else __hip_atomic_store(&s_ready[slot], kFuseNotSeeded | (j + 2u), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      const uint32_t slot = j % kFuseSlots;
      uint32_t flag = 0;
      for (uint32_t spin = 0; spin < kFuseSpin; ++spin) {
        flag = __hip_atomic_load(&s_ready[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
        if ((flag & ~kFuseNotSeeded) >= j + 1u) break;
        flag = kFuseNotSeeded;
        __builtin_amdgcn_s_sleep(2);
      }
      const uint32_t *pre = (flag & kFuseNotSeeded) ? nullptr : ring + (static_cast<size_t>(slot) * kFuseBatch + r) * kMtN;
      auto loaded = [&]() {
        if (lane == 0) __hip_atomic_fetch_add(&s_loaded[slot], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      };
      const uint32_t o = (blockIdx.x + j * gridDim.x) * kFuseBatch + r;
      if (o < n_out) walk_row(o, pre, loaded);
      else loaded();
    }
  }
}

// ---- column walk ------------------------------------------------------------------------------------
constexpr int kColThreads = 256;

template <typename T1, typename VT, int IN, int W>
__global__ __launch_bounds__(kColThreads) void jitconn_colwalk_kernel(const VT *__restrict__ in,
                                                                      T1 *__restrict__ out, uint32_t n_out,
                                                                      uint32_t n_in, uint32_t seed, double log_p,
                                                                      T1 wa, T1 wb) {
  constexpr int kWaves = kColThreads / kWave;
  constexpr int kWords = StreamLds<T1, W>::words;
  __shared__ __attribute__((aligned(8))) uint32_t s_state[kWaves * kWords];
  __shared__ uint32_t s_col[kColThreads];
  __shared__ T1 s_val[kColThreads];
  __shared__ uint32_t s_wave_cnt[kWaves];

  const int lane = lane_id();
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t c = blockIdx.x * kColThreads + threadIdx.x;
  T1 v = T1(0);
  bool on = false;
  if (c < n_in) {
    const VT x = in[c];
    on = is_event(x);
    v = static_cast<T1>(x);
  }
  const uint64_t mask = __ballot(on);
  if (lane == 0) s_wave_cnt[wave] = static_cast<uint32_t>(__popcll(mask));
  __syncthreads();
  uint32_t base = 0, count = 0;
#pragma unroll
  for (uint32_t i = 0; i < kWaves; ++i) {
    if (i < wave) base += s_wave_cnt[i];
    count += s_wave_cnt[i];
  }
  if (on) {
    const uint32_t k = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
    s_col[k] = c;
    s_val[k] = v;
  }
  __syncthreads();

  uint32_t *st = s_state + wave * kWords;
  for (uint32_t k = wave; k < count; k += kWaves) {
    const uint32_t col = s_col[k];
    const T1 val = s_val[k];
    walk_stream<T1, W>(st, lane, seed + col, nullptr, n_out, log_p, wa, wb, [&](uint32_t idx, T1 w, bool valid) {
      if (valid) {
        T1 add;
        if (IN == kInDense) add = (W == kHomo) ? val : static_cast<T1>(w * val);
        else add = w;  // homo: w == 1
        atomic_add(&out[idx], add);
      }
    });
  }
}

// Active input columns of an event vector, gathered into a list in device memory (any order): the
// column and its value.  A workgroup lists the active ones among its kCollectCols columns in LDS
// first, so that one atomic reserves all their positions (atomics of many workgroups on the one
// counter are served one after the other).
constexpr uint32_t kCollectCols = 4096;

template <typename T1, typename VT>
__global__ __launch_bounds__(1024) void collect_active_columns_kernel(const VT *__restrict__ in, uint32_t n_in,
                                                                      uint32_t *__restrict__ counter,
                                                                      uint32_t *__restrict__ list_col,
                                                                      T1 *__restrict__ list_val,
                                                                      uint32_t *__restrict__ clear, uint32_t n_clear,
                                                                      T1 *__restrict__ zero, uint32_t n_zero) {
  // (also clears the bins' counters and the output, which the kernels behind this one add to: two launches less)
  __shared__ uint32_t s_col[kCollectCols];
  __shared__ T1 s_val[kCollectCols];
  __shared__ uint32_t s_count, s_base;
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  if (tid == 0) s_count = 0;
  for (uint32_t i = blockIdx.x * 1024u + tid; i < n_clear; i += gridDim.x * 1024u) clear[i] = 0u;
  for (uint32_t i = blockIdx.x * 1024u + tid; i < n_zero; i += gridDim.x * 1024u) zero[i] = T1(0);
  __syncthreads();
  const uint32_t c0 = blockIdx.x * kCollectCols;
  for (uint32_t t = 0; t < kCollectCols; t += 1024) {
    const uint32_t c = c0 + t + tid;
    bool on = false;
    T1 v = T1(0);
    if (c < n_in) {
      const VT x = in[c];
      on = is_event(x);
      v = static_cast<T1>(x);
    }
    const uint64_t mask = __ballot(on);
    uint32_t base = 0;
    if (lane == 0 && mask) base = atomicAdd(&s_count, static_cast<uint32_t>(__popcll(mask)));
    base = __builtin_amdgcn_readfirstlane(base);
    if (on) {
      const uint32_t k = base + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
      s_col[k] = c;
      s_val[k] = v;
    }
  }
  __syncthreads();
  const uint32_t count = s_count;
  if (tid == 0) s_base = count ? atomicAdd(counter, count) : 0u;
  __syncthreads();
  const uint32_t base = s_base;
  for (uint32_t i = tid; i < count; i += 1024) {
    list_col[base + i] = s_col[i];
    list_val[base + i] = s_val[i];
  }
}

// Column walk that appends its (output, value) pairs to bins instead of adding them to `out` one
// global atomic at a time (about 21 G/s on this device).  The streams to walk are entries
// [0, n_list) of a list: column list_col[k] with value list_val[k] (event input: the active
// columns), or, without a list, column first + k with value in[first + k] (dense input).  Waves
// take entries round robin over the whole grid, so every wave walks the same number of streams.
// Not FUSED: the generators of the first n_seeded entries were seeded ahead on the vector unit (`states`);
// a wave seeding its own generator does it on the CU's one scalar unit, about 2 us each, and a
// CU's waves queue up for it.  A pair for output window b (2^shift outputs) of workgroup p goes to
// place (p * n_win + b) * cap + position of the bins; the positions continue from `counts` (zero before
// the first launch of a call), so that a call may be split into several launches; a pair that finds
// its bin full is added to `out` directly.  add_uniform_bins() then adds the bins window by window.
// The bins hold n_pairs places: `packed` (windows of at most 2^16 outputs) as an array of values with an
// array of 16-bit positions within the window behind it, 6 bytes a pair instead of 8 (10 instead of 16):
// the pairs are written once and read once, and that traffic is what a walk over a dense vector costs.
constexpr int kColBinThreads = 1024;  // 16 waves share one set of bins: 4 times fewer, 4 times larger bins
constexpr size_t kColBinBytesMax = static_cast<size_t>(3) << 30;  // bins of the dense column walk (scratch memory)

//
// FUSED: the generators are seeded inside this kernel instead, as in the row walk: workgroup p takes the
// entries p, p + G, p + 2 G, ... (G workgroups), 64 of them are a batch, its waves take (batch, entry) tasks
// from a counter in LDS, and the wave that takes the first entry of batch j first seeds batch j + 1 on the
// vector unit (lane per stream) into slot (j + 1) % 3 of the workgroup's ring of seeded states in device
// memory (`states`, kFuseRingBytes per workgroup), which the other waves read back from the L2.  Only the
// first batch of a workgroup is waited for; n_seeded is not used.
template <typename T1, typename VT, int IN, int W, bool FUSED>
__global__ __launch_bounds__(kColBinThreads, sizeof(T1) == 4 ? 8 : 4) void jitconn_colwalk_bins_kernel(
    const VT *__restrict__ in, T1 *__restrict__ out, uint32_t n_out, uint32_t seed, double log_p, T1 wa, T1 wb,
    uint32_t first, uint32_t n_list_host, const uint32_t *__restrict__ n_list_dev,
    const uint32_t *__restrict__ list_col, const T1 *__restrict__ list_val, uint32_t *states,
    uint32_t n_seeded, uint32_t n_win, uint32_t shift, uint32_t cap, void *__restrict__ pairs, uint64_t n_pairs,
    uint32_t packed, uint32_t *__restrict__ counts) {
  constexpr int kWaves = kColBinThreads / kWave;
  constexpr int kWords = StreamLds<T1, W>::words;
  __shared__ __attribute__((aligned(8))) uint32_t s_state[kWaves * kWords];
  __shared__ uint32_t s_cnt[kBinMaxWindows];
  __shared__ uint32_t s_task, s_ready[kFuseSlots], s_loaded[kFuseSlots];

  const int lane = lane_id();
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t p = blockIdx.x;
  if (threadIdx.x < n_win) s_cnt[threadIdx.x] = counts[static_cast<size_t>(threadIdx.x) * gridDim.x + p];
  if (threadIdx.x == 0) {
    s_task = 0;
    for (uint32_t k = 0; k < kFuseSlots; ++k) s_ready[k] = 0, s_loaded[k] = 0;
  }
  __syncthreads();
  const uint64_t region = static_cast<uint64_t>(p) * n_win * cap;  // first place of this workgroup's bins
  T1 *const packed_val = static_cast<T1 *>(pairs);
  uint16_t *const packed_rel = reinterpret_cast<uint16_t *>(packed_val + n_pairs);
  uint32_t *st = s_state + wave * kWords;
  const uint32_t n_list = n_list_dev ? *n_list_dev : n_list_host;

  // list entry k: its stream, seeded at `pre` (or nullptr: the wave seeds it itself)
  auto walk_entry = [&](uint32_t k, const uint32_t *pre, auto &&loaded) {
    uint32_t col;
    T1 val;
    if (list_col != nullptr) {
      col = list_col[k];
      val = list_val[k];
    } else {
      col = first + k;
      val = static_cast<T1>(in[col]);
      if (!is_event(val)) {  // a zero input adds nothing (wave uniform)
        loaded();
        return;
      }
    }
    walk_stream<T1, W>(st, lane, seed + col, pre, n_out, log_p, wa, wb, [&](uint32_t idx, T1 w, bool valid) {
      const uint32_t b = idx >> shift;
      uint32_t slot = 0;
      if constexpr (W != kNormal) {
        // The positions rise from lane to lane and the lanes that hold a synapse are the first ones of the
        // wave, so the lanes of a batch that meet in one window are neighbours (sixteen of them with
        // 16,384-output windows and conn_prob 0.001, all 64 with a dense matrix).  A returning addition
        // of several lanes to ONE counter occupies the CU's LDS for 64 cycles (measured; 7 when every lane
        // has a counter of its own), so the first lane of every run of equal windows reserves the places
        // of the whole run and the others fetch its answer (12 cycles with the shuffle): 3 to 6 % of the
        // walk, whose larger cost is the scattered stores of the pairs.  Lanes 0 and 32 begin runs of their
        // own, which keeps the masks at 32 bits.
        const uint32_t n_valid = static_cast<uint32_t>(__popcll(__ballot(valid)));
        const uint64_t heads = __ballot(b != wave_shift_up1(b)) | 0x100000001ull;
        const uint32_t half = lane < 32 ? static_cast<uint32_t>(heads) : static_cast<uint32_t>(heads >> 32);
        const uint32_t up = 31u - (static_cast<uint32_t>(lane) & 31u);  // lanes above this one in its half
        const uint32_t rank = static_cast<uint32_t>(__builtin_clz(half << up));  // lanes from the run's first to this one
        // the next run begins `run` lanes above this one (a run ends with its half at the latest)
        const uint32_t above = ((half >> 1) >> (31u - up)) | (0x80000000u >> (31u - up));
        uint32_t run = static_cast<uint32_t>(__builtin_ctz(above)) + 1u;
        if (run > n_valid - static_cast<uint32_t>(lane)) run = n_valid - static_cast<uint32_t>(lane);
        uint32_t first_slot = 0;
        if (valid && rank == 0u) first_slot = atomicAdd(&s_cnt[b], run);
        slot = static_cast<uint32_t>(__shfl(static_cast<int>(first_slot), lane - static_cast<int>(rank))) + rank;
      } else if (valid) {
        slot = atomicAdd(&s_cnt[b], 1u);  // (normal weights: the lanes that hold a synapse are not neighbours)
      }
      if (valid) {
        T1 add;
        if (IN == kInDense) add = (W == kHomo) ? val : static_cast<T1>(w * val);
        else add = w;  // homo: w == 1
        if (slot < cap) {
          const uint64_t at = region + static_cast<uint64_t>(b) * cap + slot;
          const uint32_t rel = idx & ((1u << shift) - 1u);
          if (packed) {
            packed_val[at] = add;
            packed_rel[at] = static_cast<uint16_t>(rel);
          } else {
            BinPair<T1> e;
            e.rel = rel;
            e.val = add;
            static_cast<BinPair<T1> *>(pairs)[at] = e;
          }
        } else {
          atomic_add(&out[idx], add);
        }
      }
    }, loaded);
  };

  if constexpr (!FUSED) {
    for (uint32_t k = wave * gridDim.x + p; k < n_list; k += gridDim.x * kWaves)
      walk_entry(k, (k < n_seeded) ? states + static_cast<size_t>(k) * kMtN : nullptr, NoLoadHook());
  } else {
    // this workgroup's entries: p + i * G for i < mine
    const uint32_t mine = n_list > p ? (n_list - p + gridDim.x - 1u) / gridDim.x : 0u;
    const uint32_t batches = (mine + kFuseBatch - 1u) / kFuseBatch;
    uint32_t *ring = states + static_cast<size_t>(p) * kFuseSlots * kFuseBatch * kMtN;
    auto seed_batch = [&](uint32_t j) {
      const uint32_t slot = j % kFuseSlots;
      const uint32_t i = j * kFuseBatch + static_cast<uint32_t>(lane);
      uint32_t col = 0;
      if (i < mine) {
        const uint32_t k = p + i * gridDim.x;
        col = list_col != nullptr ? list_col[k] : first + k;
      }
      const uint32_t left = mine - j * kFuseBatch;
      mt_seed_batch(st, lane, seed + col, ring + static_cast<size_t>(slot) * kFuseBatch * kMtN,
                    left < kFuseBatch ? left : kFuseBatch);
      __hip_atomic_store(&s_ready[slot], j + 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    if (wave == 0 && batches != 0) seed_batch(0);
    for (;;) {
      // (every lane adds one: the counter advances by 64 per task, any lane's old value / 64 is the task)
      const uint32_t t = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(
                             static_cast<int>(atomicAdd(&s_task, 1u)))) / kWave;
      const uint32_t j = t / kFuseBatch, r = t % kFuseBatch;
      if (j >= batches) break;
      if (r == 0 && j + 1 < batches) {
        // slot (j + 1) % 3 last held batch j - 2: (j + 1) / 3 batches have used it, 64 loads each
        const uint32_t slot = (j + 1u) % kFuseSlots, need = ((j + 1u) / kFuseSlots) * kFuseBatch;
        bool free_ = false;
        for (uint32_t spin = 0; spin < kFuseSpin && !free_; ++spin) {
          free_ = __hip_atomic_load(&s_loaded[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= need;
          if (!free_) __builtin_amdgcn_s_sleep(2);
        }
        if (free_) seed_batch(j + 1u);
        else __hip_atomic_store(&s_ready[slot], kFuseNotSeeded | (j + 2u), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      const uint32_t slot = j % kFuseSlots;
      uint32_t flag = 0;
      for (uint32_t spin = 0; spin < kFuseSpin; ++spin) {
        flag = __hip_atomic_load(&s_ready[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
        if ((flag & ~kFuseNotSeeded) >= j + 1u) break;
        flag = kFuseNotSeeded;
        __builtin_amdgcn_s_sleep(2);
      }
      const uint32_t *pre = (flag & kFuseNotSeeded) ? nullptr : ring + (static_cast<size_t>(slot) * kFuseBatch + r) * kMtN;
      auto loaded = [&]() {
        if (lane == 0) __hip_atomic_fetch_add(&s_loaded[slot], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      };
      const uint32_t i = j * kFuseBatch + r;
      if (i < mine) walk_entry(p + i * gridDim.x, pre, loaded);
      else loaded();
    }
  }
  __syncthreads();
  if (threadIdx.x < n_win) counts[static_cast<size_t>(threadIdx.x) * gridDim.x + p] = s_cnt[threadIdx.x];
}

// ---- seeding ahead ------------------------------------------------------------------------------------
constexpr int kSeedThreads = 128;

// Stream s of the launch is seed + first + s, or, with a list, seed + ids[s]; `count_dev` (optional)
// holds the number of list entries, of which at most `count` are seeded.
__global__ __launch_bounds__(kSeedThreads) void mt_seed_streams_kernel(uint32_t seed, uint32_t first, uint32_t count,
                                                                      uint32_t *__restrict__ states,
                                                                      const uint32_t *__restrict__ ids,
                                                                      const uint32_t *__restrict__ count_dev) {
  __shared__ uint32_t s_tile[kSeedThreads / kWave][kMtSeedTileWords];
  const int lane = lane_id();
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t base = (blockIdx.x * (kSeedThreads / kWave) + wave) * kWave;  // first stream of this wave
  if (count_dev != nullptr && *count_dev < count) count = *count_dev;
  if (base >= count) return;
  const uint32_t mine = base + static_cast<uint32_t>(lane);  // lane l seeds stream base + l
  uint32_t x = seed + first + mine;
  if (ids != nullptr) x = seed + (mine < count ? ids[mine] : 0u);
  mt_seed_batch(s_tile[wave], lane, x, states + static_cast<size_t>(base) * kMtN,
                count - base < static_cast<uint32_t>(kWave) ? count - base : static_cast<uint32_t>(kWave));
}

}  // namespace

void launch_seed_streams(hipStream_t stream, uint32_t seed, uint32_t first, uint32_t count, uint32_t *states) {
  if (count == 0) return;
  hipLaunchKernelGGL(mt_seed_streams_kernel, dim3(div_up(count, kSeedThreads)), dim3(kSeedThreads), 0, stream, seed,
                     first, count, states, static_cast<const uint32_t *>(nullptr),
                     static_cast<const uint32_t *>(nullptr));
}

namespace {

// ---- launchers ----------------------------------------------------------------------------------------
bool valid_log_p(const char *target, double log_p) {
  if (!(log_p < 0.0) || std::isinf(log_p)) {
    set_error("%s: log_p must be finite and negative (conn_prob in (0, 1]), got %g", target, log_p);
    return false;
  }
  return true;
}

// Scratch memory of one row-walk call, taken with ONE request so that its parts cannot move apart:
//   [packed event bitmap, the coarse bitmap behind it (only where the launcher packs one)]
//   [rings of seeded generator states, kFuseRingBytes per workgroup (only from kSeedAheadMin outputs)]
struct RowwalkScratch {
  unsigned char *base = nullptr;
  size_t bitmap_bytes = 0;   // a multiple of 256
  uint32_t ring_groups = 0;  // workgroups that have a ring
  bool refused = false;      // the stream is being captured and the memory is not there yet: the call fails
  uint32_t *bitmap() const { return bitmap_bytes && base ? reinterpret_cast<uint32_t *>(base) : nullptr; }
  uint32_t *rings() const { return ring_groups && base ? reinterpret_cast<uint32_t *>(base + bitmap_bytes) : nullptr; }
};

// At most four row-walk workgroups share a CU (eight waves each; sixteen-wave ones two).
inline uint32_t rowwalk_max_groups() { return 4u * static_cast<uint32_t>(device_info().num_cu); }

inline RowwalkScratch rowwalk_scratch(hipStream_t stream, uint32_t n_out, size_t bitmap_bytes) {
  RowwalkScratch sc;
  sc.bitmap_bytes = (bitmap_bytes + 255) / 256 * 256;
  if (n_out >= kSeedAheadMin) {
    const uint32_t batches = div_up(n_out, kFuseBatch);
    sc.ring_groups = batches < rowwalk_max_groups() ? batches : rowwalk_max_groups();
  }
  const size_t want = sc.bitmap_bytes + sc.ring_groups * kFuseRingBytes;
  if (want == 0) return sc;
  sc.base = static_cast<unsigned char *>(stream_workspace(stream, want));
  if (sc.base == nullptr && !scratch_refused_by_capture() && sc.ring_groups != 0 && sc.bitmap_bytes != 0) {
    // no room for the rings: the bitmap alone (the waves then seed their own generators)
    bpl_clear_error();
    sc.ring_groups = 0;
    sc.base = static_cast<unsigned char *>(stream_workspace(stream, sc.bitmap_bytes));
  }
  if (sc.base == nullptr) {
    sc.refused = scratch_refused_by_capture();
    if (!sc.refused) bpl_clear_error();  // (an allocation failed: paths that need no scratch memory remain)
    sc.ring_groups = 0;
  }
  return sc;
}

template <typename T1, typename VT, int IN, int W, int BITS>
void launch_rowwalk_impl(hipStream_t stream, const VT *in, T1 *out, uint32_t n_out, uint32_t n_in, uint32_t seed,
                         double log_p, T1 wa, T1 wb, int nwaves, size_t lds_bytes, const RowwalkScratch &sc) {
  const bool fused = sc.rings() != nullptr;
  auto kernel = fused ? jitconn_rowwalk_kernel<T1, VT, IN, W, BITS, true> : jitconn_rowwalk_kernel<T1, VT, IN, W, BITS, false>;
  const int block = nwaves * kWave;
  struct Cached {
    size_t lds_bytes;
    int block;
    int per_cu;
  };
  static thread_local Cached cached_for[2] = {{~size_t(0), 0, 0}, {~size_t(0), 0, 0}};
  Cached &cached = cached_for[fused];
  if (cached.lds_bytes != lds_bytes || cached.block != block) {
    if (lds_bytes > 64 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds_bytes));
    int q = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, reinterpret_cast<const void *>(kernel), block, lds_bytes) !=
            hipSuccess || q < 1) {
      (void)hipGetLastError();
      q = 1;
    }
    cached = {lds_bytes, block, q};
  }
  const unsigned resident = static_cast<unsigned>(device_info().num_cu) * static_cast<unsigned>(cached.per_cu);
  // From kSeedAheadMin outputs the generators are seeded inside the kernel, 64 at a time on the vector
  // unit, into the workgroups' rings (one launch for the whole walk); smaller walks seed in place.
  unsigned needed = fused ? div_up(n_out, kFuseBatch) : div_up(n_out, nwaves);
  if (fused && needed > sc.ring_groups) needed = sc.ring_groups;
  const unsigned grid = needed < resident ? needed : resident;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), lds_bytes, stream, in, out, n_out, n_in, seed, log_p, wa, wb, 0u,
                     sc.rings());
}

// Event probes from an LDS bitmap when it fits beside the generator states, else from global memory.
template <typename T1, typename VT, int IN, int W>
void launch_rowwalk_plain(hipStream_t stream, const VT *in, T1 *out, uint32_t n_out, uint32_t n_in, uint32_t seed,
                          double log_p, T1 wa, T1 wb, const RowwalkScratch &sc) {
  const size_t state_bytes = StreamLds<T1, W>::words * 4;
  const size_t cap = static_cast<size_t>(160) * 1024 - 512;
  // With the generators seeded inside the kernel every workgroup has a ring of seeded states in device
  // memory: 16-wave workgroups, so that the rings in use together are half as many and stay in the L2
  // and the memory-side cache.
  const int fused_waves = sc.rings() != nullptr ? 16 : 8;
  if (IN == kInEvent) {
    const size_t bitmap = (static_cast<size_t>(n_in) + 31) / 32 * 4;
    if (bitmap + 4 * state_bytes <= cap) {
      // Small bitmaps: 8-wave workgroups, several per CU.  Large ones: one workgroup per CU with
      // as many waves as fit beside the bitmap (each wave can issue one instruction every four
      // cycles, so the number of resident waves bounds the VALU utilisation).
      int nw = fused_waves;
      if (bitmap > 16 * 1024) {
        nw = static_cast<int>((cap - bitmap) / state_bytes);
        if (nw > 16) nw = 16;
      }
      launch_rowwalk_impl<T1, VT, IN, W, 1>(stream, in, out, n_out, n_in, seed, log_p, wa, wb, nw,
                                            bitmap + nw * state_bytes, sc);
      return;
    }
  }
  launch_rowwalk_impl<T1, VT, IN, W, 0>(stream, in, out, n_out, n_in, seed, log_p, wa, wb, fused_waves,
                                        fused_waves * state_bytes, sc);
}

template <typename T1, typename VT, int IN, int W>
void launch_rowwalk(hipStream_t stream, const VT *in, T1 *out, uint32_t n_out, uint32_t n_in, uint32_t seed,
                    double log_p, T1 wa, T1 wb) {
  if (n_out == 0) return;
  constexpr bool kEvents = IN == kInEvent;
  const size_t words = (static_cast<size_t>(n_in) + 31) / 32;
  // An event bitmap that would leave room for fewer than two 16-wave workgroups per CU: two levels
  // instead, the exact bitmap packed into global memory and a coarse one made for LDS.  Wide event
  // types: the vector is packed to one bit per element once, instead of once per workgroup.
  const bool two_level = kEvents && words * 4 > kRowwalkCoarseBytes;
  const bool packed = kEvents && (two_level || sizeof(VT) > 1);
  uint32_t g = 0, off = 0, c_words = 0;
  size_t bitmap_ws = 0;
  if (two_level) {
    g = coarse_shift(n_in, kRowwalkCoarseBytes);
    off = coarse_offset_words(n_in);
    c_words = (coarse_bits(n_in, g) + 31u) / 32u;
    bitmap_ws = (static_cast<size_t>(off) + c_words + 1) * sizeof(uint32_t);
  } else if (packed) {
    bitmap_ws = (words + 1) * sizeof(uint32_t);
  }
  const RowwalkScratch sc = rowwalk_scratch(stream, n_out, bitmap_ws);
  if (sc.refused) return;  // (the error stands: a graph must not record a slower path)
  if constexpr (kEvents) {
    if (uint32_t *bits = sc.bitmap()) {
      pack_event_bitmap<VT>(stream, in, n_in, bits);
      const PackedBits *pin = reinterpret_cast<const PackedBits *>(bits);
      if (two_level) {
        hipLaunchKernelGGL(coarsen_bitmap_kernel, dim3(div_up(c_words, 256)), dim3(256), 0, stream, bits,
                           static_cast<uint32_t>(words), g, bits + off, c_words);
        const size_t state_bytes = StreamLds<T1, W>::words * 4;
        launch_rowwalk_impl<T1, PackedBits, IN, W, 2>(stream, pin, out, n_out, n_in, seed, log_p, wa, wb, 16,
                                                      static_cast<size_t>(c_words) * 4 + 16 * state_bytes, sc);
      } else {
        launch_rowwalk_plain<T1, PackedBits, IN, W>(stream, pin, out, n_out, n_in, seed, log_p, wa, wb, sc);
      }
      return;
    }
  }
  launch_rowwalk_plain<T1, VT, IN, W>(stream, in, out, n_out, n_in, seed, log_p, wa, wb, sc);
}

template <typename T1, typename VT, int IN, int W>
void launch_colwalk(hipStream_t stream, const VT *in, T1 *out, uint32_t n_out, uint32_t n_in, uint32_t seed,
                    double log_p, T1 wa, T1 wb) {
  if (n_in == 0 || n_out == 0) {
    fill_zero(stream, out, n_out);
    return;
  }
  bool out_cleared = false;  // (with event input and bins, the kernel that lists the active columns clears it)
  // Many pairs: bins (also for a narrow output: seeding on the vector unit and the even spread of the streams pay).  The number of pairs is n_in * n_out * p for a
  // dense input; for events it depends on the activity, which the host does not know: bins are sized
  // for one column in eight being active (fuller bins overflow into direct atomics) and used when
  // one active column in a hundred already means a hundred thousand pairs (10,000 x 10,000 with
  // conn_prob 0.1: 44, 54 and 61 us at 0.1, 1 and 20 % activity; without bins 40, 44 and 152 us).
  const uint32_t shift = bin_window_shift(n_out);
  const uint32_t n_win = div_up(n_out, 1u << shift);
  const double p_conn = -std::expm1(log_p);
  const double full = static_cast<double>(n_in) * static_cast<double>(n_out) * p_conn;
  const bool bins = n_win <= kBinMaxWindows && full >= (IN == kInDense ? 1048576.0 : 1.0e7);
  // Event input and fewer pairs: the same list of active columns and the same seeding on the vector unit, but
  // the walk adds its pairs to `out` with atomics.  (A wave that seeds its own stream spends 2 us of the CU's one
  // scalar unit on it: with 200,000 active columns of ten synapses each the walk without a list took 1.2 ms.)
  // A dense input with fewer pairs takes the same walk over all its columns, chunk by chunk (4,000 x
  // 4,000 with conn_prob 0.02: 0.5 ms where every lane seeded the generator of its own column).
  // (Event input with fewer than 2,048 columns stays with the walk below: at 1 % activity its one launch takes 26 us
  // against the 35 us of list, seeds and walk, though 125 against 47 us at 20 %.)
  const bool listed = !bins && (IN == kInDense || n_in >= 2048);
  if (bins || listed) {
    const uint32_t n_win = bins ? div_up(n_out, 1u << bin_window_shift(n_out)) : 1u;  // (no bins: every pair overflows)
    const uint32_t shift = bins ? bin_window_shift(n_out) : 31u;
    uint32_t producers = 2u * static_cast<uint32_t>(device_info().num_cu);
    if (producers > div_up(n_in, kColBinThreads / kWave)) producers = div_up(n_in, kColBinThreads / kWave);
    auto round_up = [](size_t v) { return (v + 255) / 256 * 256; };
    // Dense input: the bins are emptied (added to `out`) after every `group` chunks of kSeedChunk columns,
    // the largest number of chunks whose pairs fit kColBinBytesMax of scratch memory (every column of a
    // 1,000,000 x 1,000,000 matrix with conn_prob 0.001 at once would take 10.7 GB).
    const bool packed = shift <= 16;
    const size_t pair_size = packed ? sizeof(T1) + 2 : sizeof(BinPair<T1>);
    const uint32_t chunks = div_up(n_in, kSeedChunk);
    uint32_t group = chunks;
    double cap_d = 0.0;
    size_t pair_bytes = 0;
    for (;;) {
      const double share = (group >= chunks) ? 1.0 : static_cast<double>(group) * kSeedChunk / static_cast<double>(n_in);
      const double per_bin = full * share / (static_cast<double>(producers) * n_win);  // every column active
      cap_d = 1.25 * per_bin + 6.0 * std::sqrt(per_bin) + 128.0;
      if (IN == kInEvent) cap_d = cap_d / 8.0 < 512.0 ? 512.0 : cap_d / 8.0;
      cap_d = std::floor(cap_d / 4.0) * 4.0;  // (packed bins begin at multiples of four places)
      pair_bytes = round_up(static_cast<size_t>(producers) * n_win * static_cast<size_t>(cap_d) * pair_size);
      if (IN == kInEvent || group == 1 || pair_bytes <= kColBinBytesMax) break;
      group = (group + 1u) / 2u;
    }
    // no bins (every pair goes to `out` with an atomic): nothing to size and nothing to empty between the chunks
    if (!bins) cap_d = 0.0, pair_bytes = 0, group = chunks;
    const size_t count_bytes = round_up(static_cast<size_t>(n_win) * producers * sizeof(uint32_t));
    // the workgroups' rings of generator states, seeded inside the walk
    const size_t state_bytes = round_up(static_cast<size_t>(producers) * kFuseRingBytes);
    const size_t list_bytes = (IN == kInEvent) ? round_up(static_cast<size_t>(n_in) * 4) : 0;
    const size_t val_bytes = (IN == kInEvent) ? round_up(static_cast<size_t>(n_in) * sizeof(T1)) : 0;
    uint32_t *list_count = (IN == kInEvent) ? stream_counters(stream) : nullptr;
    if (cap_d < 4.0e9 && pair_bytes <= (static_cast<size_t>(32) << 30) && (IN == kInDense || list_count != nullptr)) {
      const uint32_t cap = static_cast<uint32_t>(cap_d);
      unsigned char *ws = static_cast<unsigned char *>(
        stream_workspace(stream, pair_bytes + count_bytes + state_bytes + list_bytes + val_bytes));
      if (ws != nullptr) {
        void *pairs = ws;
        const uint64_t n_pairs = static_cast<uint64_t>(producers) * n_win * cap;
        uint32_t *counts = reinterpret_cast<uint32_t *>(ws + pair_bytes);
        uint32_t *states = reinterpret_cast<uint32_t *>(ws + pair_bytes + count_bytes);
        uint32_t *list_col = list_bytes ? reinterpret_cast<uint32_t *>(ws + pair_bytes + count_bytes + state_bytes) : nullptr;
        T1 *list_val = val_bytes ? reinterpret_cast<T1 *>(ws + pair_bytes + count_bytes + state_bytes + list_bytes) : nullptr;
        auto walk = jitconn_colwalk_bins_kernel<T1, VT, IN, W, true>;
        out_cleared = true;
        if (IN == kInEvent) {
          // the active columns, then one walk that seeds their generators as it goes
          hipLaunchKernelGGL((collect_active_columns_kernel<T1, VT>), dim3(div_up(n_in, kCollectCols)), dim3(1024), 0, stream,
                             in, n_in, list_count, list_col, list_val, counts, n_win * producers, out, n_out);
          hipLaunchKernelGGL(walk, dim3(producers), dim3(kColBinThreads), 0, stream, in, out, n_out, seed, log_p, wa, wb,
                             0u, 0u, static_cast<const uint32_t *>(list_count), static_cast<const uint32_t *>(list_col),
                             static_cast<const T1 *>(list_val), states, 0u, n_win, shift, cap, pairs, n_pairs, packed ? 1u : 0u, counts);
        } else {
          // every column, a chunk at a time; the bins are emptied after every `group` chunks
          fill_zero(stream, out, n_out);
          fill_zero(stream, counts, n_win * producers);
          uint32_t in_bins = 0;
          for (uint32_t first = 0; first < n_in; first += kSeedChunk) {
            const uint32_t count = (n_in - first < kSeedChunk) ? n_in - first : kSeedChunk;
            hipLaunchKernelGGL(walk, dim3(producers), dim3(kColBinThreads), 0, stream, in, out, n_out, seed, log_p, wa,
                               wb, first, count, static_cast<const uint32_t *>(nullptr),
                               static_cast<const uint32_t *>(nullptr), static_cast<const T1 *>(nullptr), states, 0u,
                               n_win, shift, cap, pairs, n_pairs, packed ? 1u : 0u, counts);
            if (++in_bins == group && first + kSeedChunk < n_in) {
              if (!add_uniform_bins<T1>("jitconn column walk", stream, out, n_out, shift, producers, cap, pairs, packed, counts,
                                        static_cast<uint32_t *>(nullptr)))
                return;  // (the error stands: part of the pairs is in `out` already)
              fill_zero(stream, counts, n_win * producers);
              in_bins = 0;
            }
          }
        }
        if (!bins) {
          if (list_count != nullptr) fill_zero(stream, list_count, 1u);  // (the list's counter goes back to zero for the next call)
          return;
        }
        if (add_uniform_bins<T1>("jitconn column walk", stream, out, n_out, shift, producers, cap, pairs, packed, counts, list_count))
          return;
        // (the bins could not be added: nothing reached `out` yet except overflow pairs; start over)
        if (list_count != nullptr) fill_zero(stream, list_count, 1u);
        out_cleared = false;
      } else {
        if (scratch_refused_by_capture()) return ensure_error("jitconn column walk", "nothing was enqueued: the path that the scratch memory at hand allows could not be launched");
        bpl_clear_error();
      }
    }
  }
  if (!out_cleared) fill_zero(stream, out, n_out);
  hipLaunchKernelGGL((jitconn_colwalk_kernel<T1, VT, IN, W>), dim3(div_up(n_in, kColThreads)), dim3(kColThreads), 0,
                     stream, in, out, n_out, n_in, seed, log_p, wa, wb);
}

// buffers = [input, out].  RAW_PROB: the descriptor's probability field holds conn_prob itself, as the
// reference packs it for its first-generation dense-vector targets (matvec.py:338-343); the walk then uses
// the log_p its CPU path derives from it (matvec.py:298), so that both versions give one matrix.
template <typename T1, typename VT, int IN, int W, bool COLWALK, bool RAW_PROB = false>
void jitconn_entry(const char *target, hipStream_t stream, void **buffers, const char *opaque, size_t opaque_len) {
  uint32_t n_row, n_col, seed;
  double log_p, a = 0, b = 0;
  if (W == kHomo) {
    bpl_jitconn_prob_homo_descriptor d;
    if (!unpack(target, opaque, opaque_len, &d)) return;
    n_row = d.n_row, n_col = d.n_col, seed = d.seed, log_p = d.log_p;
  } else {
    bpl_jitconn_prob_weight_descriptor d;
    if (!unpack(target, opaque, opaque_len, &d)) return;
    n_row = d.n_row, n_col = d.n_col, seed = d.seed, log_p = d.log_p, a = d.w_a, b = d.w_b;
  }
  if (RAW_PROB) {
    const double p = log_p;
    if (!(p > 0.0) || std::isinf(p)) {
      set_error("%s: conn_prob must be in (0, 1], got %g", target, p);
      return;
    }
    log_p = std::log(p < 1.0 ? 1.0 - p : 1e-40);
  }
  if (!valid_log_p(target, log_p)) return;
  if (buffers == nullptr) {
    set_error("%s: null buffer table", target);
    return;
  }
  const VT *in = static_cast<const VT *>(buffers[0]);
  T1 *out = static_cast<T1 *>(buffers[1]);
  if (COLWALK) launch_colwalk<T1, VT, IN, W>(stream, in, out, n_row, n_col, seed, log_p, static_cast<T1>(a), static_cast<T1>(b));
  else launch_rowwalk<T1, VT, IN, W>(stream, in, out, n_row, n_col, seed, log_p, static_cast<T1>(a), static_cast<T1>(b));
  check_launch(target);
}

// ---- self-check of the skip computation -------------------------------------------------------------
// Draw t of the check: mode 0, two hashed words; mode 1, the canonical value next to a ceil() boundary:
// U * 2^64 = exp(k * log_p) * 2^64 + j * 2^11 for k = t / 64 + 1, j = t % 64 - 32 (2^11: one unit in the
// last place of a double in [0.5, 1)).
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

__global__ __launch_bounds__(256) void check_skips_kernel(uint32_t seed, uint64_t n, int mode, double log_p,
                                                          unsigned long long *__restrict__ counts) {
  const SkipParams sp = make_skip_params(log_p);
  unsigned long long differ = 0, untrusted = 0;
  for (uint64_t t = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x; t < n;
       t += static_cast<uint64_t>(gridDim.x) * 256u) {
    uint64_t bits;
    if (mode == 0) {
      bits = mix64(t + (static_cast<uint64_t>(seed) << 32));
    } else {
      const double edge = exp(static_cast<double>(t / 64u + 1u) * log_p) * 0x1p64;
      bits = (edge < 0x1p64 ? static_cast<uint64_t>(edge) : ~0ull) +
             static_cast<uint64_t>((static_cast<int64_t>(t % 64u) - 32) * 2048);
    }
    const uint32_t lo = static_cast<uint32_t>(bits), hi = static_cast<uint32_t>(bits >> 32);
    bool safe;
    const uint32_t fast = skip_fast(lo, hi, sp, safe);
    const uint32_t exact = skip_exact(lo, hi, sp);
    if (!safe) ++untrusted;
    else if (fast != exact) ++differ;
  }
  if (differ) atomicAdd(&counts[0], differ);
  if (untrusted) atomicAdd(&counts[1], untrusted);
}

// |hardware log2 - log2| over every fp32 in [0.5, 1): the largest, as the bits of a double
__global__ __launch_bounds__(256) void check_log2_kernel(unsigned long long *__restrict__ worst) {
  const uint32_t t = blockIdx.x * 256u + threadIdx.x;  // < 2^23
  const float m = __uint_as_float(0x3f000000u | t);
  const double err = fabs(static_cast<double>(__log2f(m)) - log2(static_cast<double>(m)));
  double wave_worst = err;
  for (int d = kWave / 2; d > 0; d >>= 1) wave_worst = fmax(wave_worst, __shfl_xor(wave_worst, d, kWave));
  if (lane_id() == 0) atomicMax(worst, static_cast<unsigned long long>(__double_as_longlong(wave_worst)));
  if (t == 0) worst[1] = static_cast<unsigned long long>(__double_as_longlong(kSkipLog2Error));
}

}  // namespace

void jitconn_seed_streams(hipStream_t stream, uint32_t seed, uint32_t first, uint32_t count, uint32_t *states) {
  launch_seed_streams(stream, seed, first, count, states);
}

}  // namespace bpl

using namespace bpl;

extern "C" int bpl_selfcheck_jitconn_skips(bpl_stream_t stream, uint32_t seed, uint64_t n_draws, int near_boundaries,
                                           double log_p, uint64_t *counts) {
  if (counts == nullptr || !(log_p < 0.0)) {
    set_error("bpl_selfcheck_jitconn_skips: counts must be device memory for four words and log_p negative");
    return 1;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  unsigned long long *c = reinterpret_cast<unsigned long long *>(counts);
  hipLaunchKernelGGL(check_skips_kernel, dim3(2048), dim3(256), 0, s, seed, n_draws, near_boundaries ? 1 : 0, log_p, c);
  hipLaunchKernelGGL(check_log2_kernel, dim3((1u << 23) / 256u), dim3(256), 0, s, c + 2);
  return check_launch("bpl_selfcheck_jitconn_skips") ? 0 : 1;
}

#define BPL_DEFINE(name, ...)                                                                      \
  extern "C" void name(bpl_stream_t stream, void **buffers, const char *opaque, size_t opaque_len) { \
    jitconn_entry<__VA_ARGS__>(__func__, static_cast<hipStream_t>(stream), buffers, opaque, opaque_len); \
  }

// event input: <result type, event type, kInEvent, weight kind, column walk>
#define BPL_EVENT_FAMILY(wname, W)                                                                           \
  BPL_DEFINE(gpu_event_matvec_prob_##wname##_v2_float_bool, float, uint8_t, kInEvent, W, false)               \
  BPL_DEFINE(gpu_event_matvec_prob_##wname##_v2_float_float, float, float, kInEvent, W, false)                \
  BPL_DEFINE(gpu_event_matvec_prob_##wname##_v2_double_bool, double, uint8_t, kInEvent, W, false)             \
  BPL_DEFINE(gpu_event_matvec_prob_##wname##_v2_double_double, double, double, kInEvent, W, false)            \
  BPL_DEFINE(gpu_event_matvec_atomic_prob_##wname##_v2_float_bool, float, uint8_t, kInEvent, W, true)         \
  BPL_DEFINE(gpu_event_matvec_atomic_prob_##wname##_v2_float_float, float, float, kInEvent, W, true)          \
  BPL_DEFINE(gpu_event_matvec_atomic_prob_##wname##_v2_double_bool, double, uint8_t, kInEvent, W, true)       \
  BPL_DEFINE(gpu_event_matvec_atomic_prob_##wname##_v2_double_double, double, double, kInEvent, W, true)

#define BPL_DENSE_FAMILY(wname, W)                                                           \
  BPL_DEFINE(gpu_matvec_prob_##wname##_v2_float, float, float, kInDense, W, false)            \
  BPL_DEFINE(gpu_matvec_prob_##wname##_v2_double, double, double, kInDense, W, false)         \
  BPL_DEFINE(gpu_matvec_atomic_prob_##wname##_v2_float, float, float, kInDense, W, true)      \
  BPL_DEFINE(gpu_matvec_atomic_prob_##wname##_v2_double, double, double, kInDense, W, true)

// the reference's first-generation names (lib/gpu_ops.cc:143-148): row walk only, conn_prob in the descriptor
#define BPL_DENSE_V1_FAMILY(wname, W)                                                        \
  BPL_DEFINE(gpu_matvec_prob_##wname##_v1_float, float, float, kInDense, W, false, true)      \
  BPL_DEFINE(gpu_matvec_prob_##wname##_v1_double, double, double, kInDense, W, false, true)

BPL_EVENT_FAMILY(homo, kHomo)
BPL_EVENT_FAMILY(uniform, kUniform)
BPL_DENSE_FAMILY(homo, kHomo)
BPL_DENSE_FAMILY(uniform, kUniform)
BPL_EVENT_FAMILY(normal, kNormal)
BPL_DENSE_FAMILY(normal, kNormal)
BPL_DENSE_V1_FAMILY(homo, kHomo)
BPL_DENSE_V1_FAMILY(uniform, kUniform)
BPL_DENSE_V1_FAMILY(normal, kNormal)
