"""Benchmark of the event-driven sparse operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-extra] [--skip-cpu]

A step is one event_csr_matvec call over the 100,000 x 100,000, ~1e8-nnz heterogeneous-weight
matrix with 5 % of the event vector active, in the row-gather orientation (transpose=False),
which streams all 1e8 column indices: that is the kernel the HBM roofline applies to.  Inputs
are resident in HBM before the timed region.  The JSON line also carries, under "extra", the
scatter orientation (transpose=True) of the same matrix, the 4,000-neuron configuration, and
csr_matvec at ~1e8 nnz.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
# Counter readings cannot be taken in-process: the figures that come from rocprofv3 --pmc runs are kept in
# this file together with the kernel name, the workload, the kernel duration and the git revision they were
# taken at, and are only emitted while the run's own timing still agrees with them.
RECORDED_COUNTERS = os.path.join(ROOT, "profiles", "recorded_counters.json")
BENCH_SRC = os.path.join(ROOT, "bench_kernels.hip")
BENCH_LIB = os.path.join(ROOT, "libbench_kernels.so")


def log(*a):
  print(*a, file=sys.stderr, flush=True)


def build_kernels(force=False):
  """Compiles bench_kernels.hip (the measurement kernels: flat gather, plain stream) for gfx950."""
  from brainpylib_amd import build as b
  if force or b._newer(BENCH_LIB, [BENCH_SRC]):
    b._run([b.HIPCC] + b.HIP_FLAGS + ["-shared", BENCH_SRC, "-o", BENCH_LIB])
  return BENCH_LIB


def load_kernels():
  import ctypes
  if not os.path.exists(BENCH_LIB):
    build_kernels()
  lib = ctypes.CDLL(BENCH_LIB)
  vp, u64, i = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int
  lib.bench_gather_fma.argtypes = [vp, vp, vp, vp, vp, u64, i, i, i]
  lib.bench_gather_fma.restype = i
  lib.bench_gather_fma4.argtypes = [vp, vp, vp, vp, vp, u64, i, i, i, i, i]
  lib.bench_gather_fma4.restype = i
  lib.bench_stream.argtypes = [vp, vp, vp, u64, i, i, i]
  lib.bench_stream.restype = i
  u32 = ctypes.c_uint32
  lib.bench_lds_atomic.argtypes = [vp, vp, i, i, i]
  lib.bench_lds_atomic.restype = i
  lib.bench_global_atomic.argtypes = [vp, vp, u32, i, i, i]
  lib.bench_global_atomic.restype = i
  lib.bench_l2_read.argtypes = [vp, vp, vp, u32, i, i]
  lib.bench_l2_read.restype = i
  return lib


def recorded_counters(key, kernel_us, tolerance=0.05, **must_match):
  """The entry `key` of profiles/recorded_counters.json if it still describes this run: the fields in
  `must_match` are equal and the kernel's duration measured now is within `tolerance` of the one at
  which the counters were read.  Else None (and the reason on stderr)."""
  try:
    with open(RECORDED_COUNTERS) as f:
      entry = json.load(f)[key]
  except (OSError, KeyError, ValueError) as e:
    log("recorded counters: no usable entry %r (%s)" % (key, e))
    return None
  for k, v in must_match.items():
    if entry.get(k) != v:
      log("recorded counters %r: %s is %r there, %r here: not used" % (key, k, entry.get(k), v))
      return None
  if abs(kernel_us - entry["kernel_us"]) > tolerance * entry["kernel_us"]:
    log("recorded counters %r: kernel took %.1f us when they were read, %.1f us now: not used" % (
      key, entry["kernel_us"], kernel_us))
    return None
  return entry


# The device raises its clocks only under sustained load: for the first 50-100 ms after an idle spell (a host-side
# oracle computation, say) kernels that are bound by instruction issue run 15-20 % slower (jitconn matmat: 285 us
# against 240 us from the hundredth call on).  Every timed region is therefore preceded by at least this much
# untimed work of the same kind, beyond the W warm-up calls asked for.
CLOCK_WARM_S = 0.15


def time_calls(fn, steps, warmup, warm_s=None):
  """Per-call GPU durations (HIP events on the stream the kernels are enqueued on) and the
  wall time of the K back-to-back calls.  Untimed before them: `warmup` calls, then further calls
  until `warm_s` seconds (default CLOCK_WARM_S) have passed since the first one."""
  import torch
  warm_s = CLOCK_WARM_S if warm_s is None else warm_s
  tw = time.perf_counter()
  for _ in range(warmup):
    fn()
  torch.cuda.synchronize()
  while time.perf_counter() - tw < warm_s:
    for _ in range(4):
      fn()
    torch.cuda.synchronize()
  starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
  ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
  t0 = time.perf_counter()
  for i in range(steps):
    starts[i].record()
    fn()
    ends[i].record()
  torch.cuda.synchronize()
  wall = time.perf_counter() - t0
  dur_ms = np.array([s.elapsed_time(e) for s, e in zip(starts, ends)])
  return dur_ms, wall


def single_call_us(fn, reps=20):
  """Wall microseconds of ONE call with an idle queue before it and a synchronize after it: launch,
  the kernels and the wait, as a caller that needs the result at once pays them.  Returns the first
  (cold: whatever this call is the first to touch is loaded or allocated inside it) and the median
  of `reps` further ones."""
  import torch
  out = []
  for _ in range(reps + 1):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    out.append((time.perf_counter() - t0) * 1e6)
  return dict(first=out[0], median=float(np.median(out[1:])))


def copy_bandwidth_gb_per_s(dev, n_bytes=1 << 30):
  """What a plain device-to-device copy of `n_bytes` moves per second on this device (bytes read
  plus bytes written): the HBM rate a streaming kernel can actually reach, to set beside the
  published peak."""
  import torch
  a = torch.empty(n_bytes // 4, dtype=torch.float32, device=dev).normal_()
  b = torch.empty_like(a)
  dur, _ = time_calls(lambda: b.copy_(a), 20, 3)
  return 2.0 * n_bytes / (float(np.median(dur)) * 1e-3) / 1e9


def gather_ceiling(lib, dev, x, idx, w, steps):
  """What a kernel that does csr_matvec's work per nonzero WITHOUT the row structure reaches on this
  device: acc += x[idx[j]] * w[j] over the flat index and weight streams (two coalesced streams, one
  random 4-byte read of the vector per nonzero), at the occupancies and numbers of loads in flight a CSR
  product can run with, the streams read 4 bytes per lane or 16 bytes per lane with the nontemporal hint.
  The best rate is the ceiling of any product that gathers the vector from L2."""
  import ctypes
  import torch
  n = int(idx.numel())
  cu = torch.cuda.get_device_properties(dev).multi_processor_count
  stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  rows = []
  for per_cu, threads, inflight in ((2, 1024, 4), (2, 1024, 8), (1, 1024, 8), (4, 512, 8), (8, 256, 8)):
    blocks = cu * per_cu
    out = torch.zeros(blocks * threads, dtype=torch.float32, device=dev)
    fn = lambda: lib.bench_gather_fma(stream, x.data_ptr(), idx.data_ptr(), w.data_ptr(), out.data_ptr(), n, blocks,
                                      threads, inflight)
    if fn() != 0:
      raise SystemExit("bench_gather_fma failed to launch")
    d, _ = time_calls(fn, steps, 2)
    rows.append(dict(stream_loads="4 bytes", workgroups_per_cu=per_cu, threads=threads, loads_in_flight=inflight,
                     us=float(d.mean() * 1e3), g_gathers_per_s=n / (d.mean() * 1e-3) / 1e9,
                     checksum=float(out.double().sum().item())))
  n4 = n - n % 4
  for per_cu, threads, quads, pieces in ((2, 1024, 4, 1), (1, 1024, 4, 1), (2, 512, 4, 1), (2, 512, 4, 8), (4, 512, 2, 1)):
    blocks = cu * per_cu
    out = torch.zeros(blocks * threads, dtype=torch.float32, device=dev)
    fn = lambda: lib.bench_gather_fma4(stream, x.data_ptr(), idx.data_ptr(), w.data_ptr(), out.data_ptr(), n4, blocks,
                                       threads, quads, 1, pieces)
    if fn() != 0:
      raise SystemExit("bench_gather_fma4 failed to launch")
    d, _ = time_calls(fn, steps, 2)
    tail = float((x[idx[n4:].long()].double() * w[n4:].double()).sum().item())
    rows.append(dict(stream_loads="16 bytes, nontemporal, %d piece(s) per instruction" % pieces, workgroups_per_cu=per_cu,
                     threads=threads, loads_in_flight=4 * quads, us=float(d.mean() * 1e3),
                     g_gathers_per_s=n4 / (d.mean() * 1e-3) / 1e9, checksum=float(out.double().sum().item()) + tail))
  return rows


def stream_ceiling(lib, dev, n_bytes, steps):
  """GB/s of 16-byte loads, plain and nontemporal, over `n_bytes` of HBM at a persistent kernel's occupancies:
  the read rate a streaming kernel reaches on this device (the published peak is not reachable by any kernel)."""
  import ctypes
  import torch
  n16 = n_bytes // 16
  buf = torch.empty(n16 * 4, dtype=torch.int32, device=dev).random_()
  cu = torch.cuda.get_device_properties(dev).multi_processor_count
  stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  rows = []
  for nt in (0, 1):
    for per_cu, threads in ((2, 1024), (1, 1024), (4, 512), (8, 256)):
      blocks = cu * per_cu
      out = torch.zeros(blocks * threads, dtype=torch.int32, device=dev)
      fn = lambda: lib.bench_stream(stream, buf.data_ptr(), out.data_ptr(), n16, blocks, threads, nt)
      if fn() != 0:
        raise SystemExit("bench_stream failed to launch")
      d, _ = time_calls(fn, steps, 2)
      rows.append(dict(workgroups_per_cu=per_cu, threads=threads, nontemporal=bool(nt), us=float(d.mean() * 1e3),
                       gb_per_s=n16 * 16 / (d.mean() * 1e-3) / 1e9))
  return rows


def back_to_back_us(fn, calls):
  """Microseconds per call when `calls` calls are enqueued with nothing between them (one pair of
  events around all of them): what a time-stepping loop pays per call once the queue is fed."""
  import torch
  for _ in range(20):
    fn()
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(calls):
    fn()
  e1.record()
  torch.cuda.synchronize()
  return e0.elapsed_time(e1) * 1e3 / calls


def stats(dur_ms):
  return dict(mean_us=float(dur_ms.mean() * 1e3), median_us=float(np.median(dur_ms) * 1e3),
              p95_us=float(np.percentile(dur_ms, 95) * 1e3), min_us=float(dur_ms.min() * 1e3))


def check(got, want, what, mag=None):
  """Parity gate.  The bound is rel 1e-5 / abs 1e-6; sums accumulated in another order than the oracle's
  sequential loop (`mag` = sum of |addends| per element) may additionally differ by the reordering bound
  4 eps sum|addends|.  Both counts are printed: elements outside the plain bound, and violations of the gate."""
  got = np.asarray(got, dtype=np.float64)
  want = np.asarray(want, dtype=np.float64)
  plain = 1e-6 + 1e-5 * np.abs(want)
  bound = plain
  if mag is not None:
    bound = plain + 4 * np.finfo(np.float32).eps * np.asarray(mag, dtype=np.float64)
  err = np.abs(got - want)
  bad = int((err > bound).sum())
  outside_plain = int((err > plain).sum())
  log("parity %-34s max abs err %.3e  outside rel 1e-5/abs 1e-6: %d  violations%s: %d / %d" % (
    what, float(err.max(initial=0)), outside_plain, " (with reordering term)" if mag is not None else "", bad, got.size))
  if bad:
    raise SystemExit("parity gate failed for " + what)
  return outside_plain


def parity_record(got, outside_plain, bound):
  """What a leg says about its parity gate: how many elements were compared, how many of them lay outside the
  plain rel 1e-5 / abs 1e-6 bound (and passed through the reordering term only), violations (always 0: a
  violation ends the run), and which bound applied."""
  return dict(elements=int(np.asarray(got).size), outside_plain=int(outside_plain), violations=0, bound=bound)


def roofline_record(bound, achieved, peak, unit, **more):
  return dict(bound=bound, achieved=float(achieved), peak=float(peak), unit=unit, frac=float(achieved) / float(peak), **more)


def device_rates(lib, dev):
  """Rates of the device's building blocks that the kernels' designs are argued from, measured in this run:
  LDS read-modify-writes by type, atomic adds in device memory (random addresses; one address), and the rate at
  which the L2s deliver lines of a buffer that stays resident in them.  A few milliseconds in all."""
  import ctypes
  import torch
  stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  cu = torch.cuda.get_device_properties(dev).multi_processor_count
  rates = {}

  def timed(fn, reps=5):
    if fn() != 0:
      raise SystemExit("a device-rate kernel failed to launch")
    d, _ = time_calls(fn, reps, 2, warm_s=0.05)
    return float(np.median(d)) * 1e-3  # seconds

  blocks, iters = 2 * cu, 2048
  out = torch.zeros(blocks, dtype=torch.float32, device=dev)
  ops = blocks * 1024 * iters
  for mode, name in ((0, "lds_add_f32"), (1, "lds_add_u32"), (2, "lds_add_f64"), (3, "lds_write_b32"),
                     (4, "lds_address_arithmetic_only")):
    t = timed(lambda: lib.bench_lds_atomic(stream, out.data_ptr(), blocks, iters, mode))
    rates[name + "_g_per_s"] = ops / t / 1e9
  # returning additions with 1, 4 and 16 neighbouring lanes per counter: time of a CU's LDS per wave instruction (2.4 cycles per ns)
  for mode, lanes in ((101, 1), (104, 4), (116, 16)):
    t = timed(lambda: lib.bench_lds_atomic(stream, out.data_ptr(), blocks, iters, mode))
    rates["lds_returning_add_%d_lanes_per_counter_ns_per_wave_instruction_and_cu" % lanes] = t / (blocks / cu * 16 * iters) * 1e9
  rates["lds_workload"] = "%d workgroups of 1,024 threads, %d random operations per thread in a 64 KB window" % (blocks, iters)
  for n in (100_000, 1_000_000, 16_000_000):
    y = torch.zeros(n, dtype=torch.float32, device=dev)
    gb, gi = 4096, 64
    t = timed(lambda: lib.bench_global_atomic(stream, y.data_ptr(), n, gb, gi, 0))
    rates["global_atomic_add_f32_random_%d_g_per_s" % n] = gb * 256 * gi / t / 1e9
    del y
  cnt = torch.zeros(64, dtype=torch.int32, device=dev)
  sb, si = 512, 256
  t = timed(lambda: lib.bench_global_atomic(stream, cnt.data_ptr(), 1, sb, si, 1))
  rates["global_atomic_same_address_ns_each"] = t / (sb * si) * 1e9
  # 2 MB: well inside each 4 MB L2
  n16 = (2 << 20) // 16
  buf = torch.empty(n16 * 4, dtype=torch.int32, device=dev).random_()
  for per_cu in (1, 2):
    lb, reps = cu * per_cu, 16
    o2 = torch.zeros(lb * 1024, dtype=torch.int32, device=dev)
    t = timed(lambda: lib.bench_l2_read(stream, buf.data_ptr(), o2.data_ptr(), n16, reps, lb))
    rates["l2_read_2MB_%d_workgroups_per_cu_tb_per_s" % per_cu] = lb * reps * n16 * 16.0 / t / 1e12
  return rates


def reference_shapes(bpl, synth, torch, dev):
  """The reference's benchmark scripts time 100 jitted calls including dispatch on an unstated GPU; their
  docstring figures (seconds per 100 calls) are quoted as ms per call.  Ours: mean HIP-event time per call."""
  rows = []
  # event_matvec_jitconn_performance.py:157-195: homogeneous weight 1.0, FixedProb(prob), events density = prob
  ref_event = {(1000, 1000, 0.1): (0.957, 0.996, 1.294, 1.456), (10000, 10000, 0.1): (1.541, 1.557, 1.585, 1.890),
               (10000, 10000, 0.2): (2.872, 2.905, 3.945, 2.663), (50000, 50000, 0.1): (1.485, 2.521, 6.014, 5.887),
               (50000, 50000, 0.2): (4.123, 5.962, 10.801, 11.053)}
  for (n0, n1, p), (csr_t, csr_n, jit_t, jit_n) in ref_event.items():
    indices, indptr = synth.bernoulli_csr(n0, n1, p, seed=n0 + int(p * 100))
    rng = np.random.default_rng(5)
    d_idx, d_ptr = torch.from_numpy(indices).to(dev), torch.from_numpy(indptr).to(dev)
    w = torch.ones(1, dtype=torch.float32, device=dev)
    for transpose, ref_csr, ref_jit in ((True, csr_t, jit_t), (False, csr_n, jit_n)):
      ev = torch.from_numpy(rng.random(n0 if transpose else n1) < p).to(dev)
      d, _ = time_calls(lambda: bpl.event_csr_matvec(w, d_idx, d_ptr, ev, shape=(n0, n1), transpose=transpose), 100, 10)
      dj, _ = time_calls(lambda: bpl.event_matvec_prob_conn_homo_weight(ev, 1.0, conn_prob=p, shape=(n0, n1), seed=1234,
                                                                        transpose=transpose), 30, 3)
      rows.append(dict(op="event_csr_matvec homo", shape=[n0, n1], prob=p, transpose=transpose,
                       ours_ms=float(d.mean()), reference_docstring_ms=ref_csr))
      rows.append(dict(op="jitconn event_matvec homo", shape=[n0, n1], prob=p, transpose=transpose,
                       ours_ms=float(dj.mean()), reference_docstring_ms=ref_jit))
      log(rows[-2]); log(rows[-1])
    del d_idx, d_ptr
  # csr_matvec_VS_cusparse_csr_matvec.py:76-111: heterogeneous weights, FixedProb(0.1), method='vector'
  ref_csr = {(10000, 10000): 1.715, (100000, 10000): 3.428, (50000, 50000): 9.002, (100000, 50000): 16.211}
  for (n0, n1), ref_ms in ref_csr.items():
    indices, indptr = synth.bernoulli_csr(n0, n1, 0.1, seed=n0 + n1)
    rng = np.random.default_rng(6)
    d_idx, d_ptr = torch.from_numpy(indices).to(dev), torch.from_numpy(indptr).to(dev)
    data = torch.from_numpy(rng.random(indices.shape[0], dtype=np.float32)).to(dev)
    v = torch.from_numpy(rng.random(n1, dtype=np.float32)).to(dev)
    d, _ = time_calls(lambda: bpl.csr_matvec(data, d_idx, d_ptr, v, shape=(n0, n1)), 50, 5)
    rows.append(dict(op="csr_matvec heter", shape=[n0, n1], prob=0.1, nnz=int(indices.shape[0]),
                     ours_ms=float(d.mean()), reference_docstring_ms=ref_ms))
    log(rows[-1])
    del d_idx, d_ptr, data
  print(json.dumps({"reference_shapes": rows}), flush=True)


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=200)
  ap.add_argument("--warmup", type=int, default=20)
  ap.add_argument("--skip-extra", action="store_true", help="only the headline workload")
  ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU baseline")
  ap.add_argument("--pmc", choices=["gather", "scatter", "csr", "jitconn", "jitconn-normal", "jitconn-dense", "jitconn-dense-column", "matmat"],
                  default=None,
                  help="counter-collection mode for rocprofv3 --pmc.  gather: three plain copies of 400 MB "
                       "(the calibration kernel), three calls of the headline kernel and three plain streams over "
                       "740 MB.  scatter: three calls of the same matrix with transpose=True.  csr: three calls of "
                       "csr_matvec on the 1,000,000 x 1,000,000 matrix in each orientation and three flat gathers over "
                       "the same index and weight streams.  jitconn: three calls "
                       "of jitconn event matvec (1e6 x 1e6, p=0.001) in both walks.  jitconn-normal: three "
                       "row walks of the same matrix with normal weights.  jitconn-dense: three row walks over a "
                       "dense vector.  matmat: three calls of jitconn matmat 10,000 x 10,000 x 128.  Nothing else runs.")
  ap.add_argument("--rates", action="store_true",
                  help="only the device's building-block rates (LDS atomics by type, atomics in device memory, L2 line "
                       "delivery): one JSON line {\"device_rates\": ...}")
  ap.add_argument("--reference-shapes", action="store_true",
                  help="instead of the headline run: the shapes of the reference's own benchmark scripts "
                       "(event_matvec_jitconn_performance.py, csr_matvec_VS_cusparse_csr_matvec.py), with the "
                       "per-call times pasted in their docstrings beside ours")
  args = ap.parse_args()
  if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
    raise SystemExit("bench.py: this build runs on ONE GPU (the operators are single-device, like the "
                     "reference's); --gpus %d is not supported." % args.gpus)

  import torch
  import brainpylib_amd as bpl
  import benchdata as synth
  import oracle  # checker and CPU baseline only

  assert torch.cuda.is_available(), "bench.py needs a HIP device"
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  cores = len(os.sched_getaffinity(0))

  if args.reference_shapes:
    reference_shapes(bpl, synth, torch, dev)
    return

  if args.rates:
    print(json.dumps({"device_rates": device_rates(load_kernels(), dev)}), flush=True)
    return

  if args.pmc == "jitconn":
    j = synth.config_jitconn_event()
    ev = torch.from_numpy(j["events"]).to(dev)
    for odp in (True, False):
      for _ in range(3):
        bpl.event_matvec_prob_conn_homo_weight(ev, j["weight"], conn_prob=j["conn_prob"], shape=j["shape"],
                                               seed=j["seed"], outdim_parallel=odp)
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  if args.pmc in ("jitconn-dense", "jitconn-dense-column"):
    j = synth.config_jitconn_event()
    vec = torch.randn(j["shape"][0], dtype=torch.float32, device=dev)
    for _ in range(3):
      bpl.matvec_prob_conn_homo_weight(vec, j["weight"], conn_prob=j["conn_prob"], shape=j["shape"], seed=j["seed"],
                                       outdim_parallel=args.pmc == "jitconn-dense")
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  if args.pmc == "matmat":
    mm = synth.config_jitconn_matmat()
    X = torch.from_numpy(np.ascontiguousarray(mm["B"].T)).to(dev)
    for _ in range(3):
      bpl.matmat_prob_conn_normal_weight(X, w_mu=mm["w_mu"], w_sigma=mm["w_sigma"], conn_prob=mm["conn_prob"],
                                         shape=mm["shape"], seed=mm["seed"])
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  if args.pmc == "csr":
    import ctypes
    m = synth.config_csr_matvec()
    md = {k: torch.from_numpy(v).to(dev) for k, v in m.items() if isinstance(v, np.ndarray)}
    for _ in range(3):
      bpl.csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"], shape=m["shape"])
    for _ in range(3):
      bpl.cusparse_csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"], shape=m["shape"], transpose=True)
    # the transposed product whose output fits one float64 window in LDS: 1,000,000 x 16,000, 50 per row
    ix_n, ip_n = synth.counted_csr(np.full(1_000_000, 50), 16_000, seed=29)
    rng_n = np.random.default_rng(23)
    dev_n = [torch.from_numpy(a_).to(dev) for a_ in (rng_n.random(ix_n.shape[0], dtype=np.float32), ix_n, ip_n,
                                                      rng_n.standard_normal(1_000_000).astype(np.float32))]
    for _ in range(3):
      bpl.cusparse_csr_matvec(*dev_n, shape=(1_000_000, 16_000), transpose=True)
    lib = load_kernels()
    cu = torch.cuda.get_device_properties(dev).multi_processor_count
    out = torch.zeros(cu * 2 * 1024, dtype=torch.float32, device=dev)
    for _ in range(3):
      lib.bench_gather_fma(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), md["vector"].data_ptr(),
                           md["indices"].data_ptr(), md["data"].data_ptr(), out.data_ptr(), md["indices"].numel(),
                           cu * 2, 1024, 8)
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  if args.pmc == "jitconn-normal":
    j = synth.config_jitconn_event()
    ev = torch.from_numpy(j["events"]).to(dev)
    for _ in range(3):
      bpl.event_matvec_prob_conn_normal_weight(ev, w_mu=0.0, w_sigma=1.0, conn_prob=j["conn_prob"], shape=j["shape"],
                                               seed=j["seed"], outdim_parallel=True)
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  # ---------------------------------------------------------------------------------------------
  # headline workload: event_csr_matvec, 100,000 x 100,000, ~1e8 nnz, heterogeneous weights
  # ---------------------------------------------------------------------------------------------
  t0 = time.time()
  c = synth.config_event_csr_large()
  n_row, n_col = c["shape"]
  nnz = int(c["indices"].shape[0])
  log("generated event_csr_matvec workload: nnz %d in %.1f s" % (nnz, time.time() - t0))
  data = torch.from_numpy(c["data"]).to(dev)
  indices = torch.from_numpy(c["indices"]).to(dev)
  indptr = torch.from_numpy(c["indptr"]).to(dev)
  events = torch.from_numpy(c["events"]).to(dev)

  # parity gate at full size (the oracle's single-thread loops take well under a second each)
  want_g = oracle.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"])
  torch.cuda.synchronize()
  t1 = time.perf_counter()
  got_dev = bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"])
  torch.cuda.synchronize()
  cold_gather_us = (time.perf_counter() - t1) * 1e6  # this process's first call of the operator
  got_g = got_dev.cpu().numpy()
  del got_dev
  outside_g = check(got_g, want_g, "event_csr_matvec gather 1e8 nnz")
  want_s = oracle.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=True)
  mag_s = oracle.event_csr_matvec(np.abs(c["data"]), c["indices"], c["indptr"], c["events"], shape=c["shape"],
                                  transpose=True)
  got_s = bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"], transpose=True).cpu().numpy()
  outside_s = check(got_s, want_s, "event_csr_matvec scatter 1e8 nnz", mag_s)

  if args.pmc == "scatter":
    for _ in range(3):
      bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"], transpose=True)
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  if args.pmc == "gather":
    src = torch.empty(100_000_000, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(3):
      dst.copy_(src)  # reads 400,000,000 bytes and writes 400,000,000 bytes
    torch.cuda.synchronize()
    for _ in range(3):
      bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"])
    torch.cuda.synchronize()
    import ctypes
    lib = load_kernels()
    cu = torch.cuda.get_device_properties(dev).multi_processor_count
    buf = torch.empty(740_000_000 // 4, dtype=torch.int32, device=dev).random_()
    out = torch.zeros(cu * 2 * 1024, dtype=torch.int32, device=dev)
    for _ in range(3):
      lib.bench_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), buf.data_ptr(), out.data_ptr(),
                       740_000_000 // 16, cu * 2, 1024, 0)
    torch.cuda.synchronize()
    log("pmc mode done")
    return

  hits = int(c["events"][c["indices"]].sum())                 # synapses whose pre-neuron fired (gather view)
  active = int(c["events"].sum())
  delivered = int(np.diff(c["indptr"].astype(np.int64))[c["events"]].sum())  # scatter view

  def gather():
    return bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"], transpose=False)

  dur, wall = time_calls(gather, args.steps, args.warmup)
  ms_per_step = wall / args.steps * 1e3
  kernel_ms = float(dur.mean())
  # algorithmic bytes of one gather call: indptr + all indices + the data elements that are
  # hit + the event vector + the output
  bytes_gather = 4 * (n_row + 1) + 4 * nnz + 4 * hits + n_col * 1 + 4 * n_row
  achieved = bytes_gather / (kernel_ms * 1e-3) / 1e9
  value = nnz / (ms_per_step * 1e-3) / 1e9
  log("gather: %.1f us/call (events) %.1f us/step (wall)  %.1f GSOP/s  %.0f GB/s algorithmic" % (
    kernel_ms * 1e3, ms_per_step * 1e3, value, achieved))

  extra = {"gather_call_us": stats(dur), "nnz": nnz, "hits": hits, "active_rows": active,
           "gather_parity": parity_record(got_g, outside_g, "rel 1e-5 / abs 1e-6 (the row sums are formed in the "
                                                            "oracle's order in float64 and rounded once)")}
  one = single_call_us(gather)
  copy_rate = copy_bandwidth_gb_per_s(dev)
  extra["hbm_copy_gb_per_s"] = copy_rate  # 1 GiB device-to-device copy, read + write
  log("device-to-device copy of 1 GiB: %.0f GB/s (read + write)" % copy_rate)
  # what plain 16-byte loads over the same number of bytes reach at this kernel's occupancy
  bench_lib = load_kernels()
  extra["device_rates"] = device_rates(bench_lib, dev)
  log("device rates: %s" % extra["device_rates"])
  rec = recorded_counters("event_csr_gather_1e8", kernel_ms * 1e3, nnz=nnz)
  traffic = float(rec["hbm_bytes_per_launch"]) if rec else None
  streams = stream_ceiling(bench_lib, dev, int(traffic) if traffic else bytes_gather, 20)
  stream_rate = max(r["gb_per_s"] for r in streams)
  extra["hbm_stream_read"] = dict(best_gb_per_s=stream_rate, runs=streams)
  log("16-byte loads, plain and nontemporal: %s" % streams)
  if traffic:
    extra["gather_hbm_traffic_gb_per_s"] = traffic / (kernel_ms * 1e-3) / 1e9
    extra["gather_traffic_over_copy_rate"] = extra["gather_hbm_traffic_gb_per_s"] / copy_rate
  extra["gather_single_call_wall_us"] = dict(cold_first_in_process=cold_gather_us, warm_median=one["median"])

  # ---------------------------------------------------------------------------------------------
  # CPU baseline: the oracle's restatement of the reference's CPU loop for this exact call
  # (heterogeneous gather: single-threaded in the reference), bounded to ~10-20 s
  # ---------------------------------------------------------------------------------------------
  cpu_baseline = None
  if not args.skip_cpu:
    oracle.set_threads(1)
    n_cpu, t_cpu = 0, 0.0
    while t_cpu < 10.0 and n_cpu < 50:
      t1 = time.perf_counter()
      oracle.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"])
      t_cpu += time.perf_counter() - t1
      n_cpu += 1
    cpu_baseline = {"value": nnz / (t_cpu / n_cpu) / 1e9, "unit": "GSOP/s", "cores": 1, "kind": "port",
                    "sample": "%d full calls of the same workload (%.2f s each), C restatement of "
                              "event_csr_matvec.py:334-347 compiled with gcc -O2" % (n_cpu, t_cpu / n_cpu)}
    log("cpu baseline: %.3f s/call -> %.2f GSOP/s on 1 of %d cores" % (t_cpu / n_cpu, cpu_baseline["value"], cores))

  if not args.skip_extra:
    # scatter orientation of the same matrix
    def scatter():
      return bpl.event_csr_matvec(data, indices, indptr, events, shape=c["shape"], transpose=True)
    dur_s, wall_s = time_calls(scatter, args.steps, args.warmup)
    bytes_scatter = n_row * 1 + 8 * active + delivered * 8 + 4 * n_col
    extra["scatter_1e8"] = dict(stats(dur_s), delivered_synapses=delivered,
                                gsop_per_s=delivered / (dur_s.mean() * 1e-3) / 1e9,
                                algorithmic_gb_per_s=bytes_scatter / (dur_s.mean() * 1e-3) / 1e9,
                                wall_us_per_call=wall_s / args.steps * 1e6,
                                roofline=roofline_record("hbm", bytes_scatter / (dur_s.mean() * 1e-3) / 1e9, HBM_PEAK_GBS,
                                                         "GB/s", algorithmic_bytes_per_call=bytes_scatter,
                                                         launches_per_call=3),
                                parity=parity_record(got_s, outside_s, "rel 1e-5 / abs 1e-6 + 4 eps sum|addends|"))
    if not args.skip_cpu:
      t1 = time.perf_counter()
      for _ in range(20):
        oracle.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=True)
      t_cpu = (time.perf_counter() - t1) / 20
      extra["scatter_1e8"]["cpu_port_1core_us"] = t_cpu * 1e6
      # the reference's own compiled kernel for this orientation (lib/cpu_event_sum.cc), where it was built
      from oracle import ref
      if ref.available():
        got_ref = ref.csr_event_sum(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"])
        check(got_ref, want_s, "reference cpu_csr_event_sum_heter vs oracle (scatter 1e8 nnz)")
        t1 = time.perf_counter()
        for _ in range(20):
          ref.csr_event_sum(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"])
        extra["scatter_1e8"]["cpu_reference_1core_us"] = (time.perf_counter() - t1) / 20 * 1e6
    log("scatter 1e8: %s" % extra["scatter_1e8"])

    # homogeneous weight, gather: only the index stream is read
    w = torch.tensor([0.6], dtype=torch.float32, device=dev)
    dur_h, _ = time_calls(lambda: bpl.event_csr_matvec(w, indices, indptr, events, shape=c["shape"]), args.steps,
                          args.warmup)
    bytes_h = 4 * (n_row + 1) + 4 * nnz + n_col + 4 * n_row
    got_h = bpl.event_csr_matvec(w, indices, indptr, events, shape=c["shape"]).cpu().numpy()
    want_h = oracle.event_csr_matvec(np.array([0.6], np.float32), c["indices"], c["indptr"], c["events"], shape=c["shape"])
    if not np.array_equal(got_h, want_h):
      raise SystemExit("parity gate failed for the homogeneous gather (bit for bit)")
    extra["gather_homo_1e8"] = dict(stats(dur_h), gsop_per_s=nnz / (dur_h.mean() * 1e-3) / 1e9,
                                    algorithmic_gb_per_s=bytes_h / (dur_h.mean() * 1e-3) / 1e9,
                                    roofline=roofline_record("hbm", bytes_h / (dur_h.mean() * 1e-3) / 1e9, HBM_PEAK_GBS,
                                                             "GB/s", algorithmic_bytes_per_call=bytes_h),
                                    parity=dict(elements=int(got_h.size), outside_plain=0, violations=0,
                                                bound="bit for bit"))
    log("gather homo 1e8: %s" % extra["gather_homo_1e8"])

    # vmap over event vectors (event_csr_matvec_batching): the same matrix against 8 and 32
    # event vectors of the same rate; the index stream is read once per 8 vectors
    rng_b = np.random.default_rng(99)
    batched = {}
    for nb in (8, 32):
      evb = torch.from_numpy(rng_b.random((nb, n_col)) < 0.05).to(dev)
      dur_b, _ = time_calls(lambda: bpl.event_csr_matvec_batching(
        data[None], indices[None], indptr[None], evb, batch_size=nb, shape=c["shape"]), max(args.steps // 4, 5),
        max(args.warmup // 4, 2))
      batched["x%d" % nb] = dict(stats(dur_b), us_per_event_vector=float(dur_b.mean() * 1e3 / nb),
                                 gsop_per_s=nb * nnz / (dur_b.mean() * 1e-3) / 1e9)
      del evb
    extra["gather_batched_1e8"] = batched
    log("gather batched 1e8: %s" % batched)
    # the same in scatter orientation: 8 event vectors of 1 % and 5 % activity through one sorted scatter
    batched_t = {}
    for rate in (0.01, 0.05):
      ev_np = rng_b.random((8, n_row)) < rate
      evb = torch.from_numpy(ev_np).to(dev)
      got = bpl.event_csr_matvec_batching(data[None], indices[None], indptr[None], evb, batch_size=8, shape=c["shape"],
                                          transpose=True)[3].cpu().numpy()
      want = oracle.event_csr_matvec(c["data"], c["indices"], c["indptr"], ev_np[3], shape=c["shape"], transpose=True)
      mag = oracle.event_csr_matvec(np.abs(c["data"]), c["indices"], c["indptr"], ev_np[3], shape=c["shape"],
                                    transpose=True)
      check(got, want, "batched scatter 1e8 nnz, entry 3 at %g" % rate, mag)
      dur_b, _ = time_calls(lambda: bpl.event_csr_matvec_batching(
        data[None], indices[None], indptr[None], evb, batch_size=8, shape=c["shape"], transpose=True),
        max(args.steps // 4, 5), max(args.warmup // 4, 2))
      batched_t["x8_events_%g" % rate] = dict(stats(dur_b), us_per_event_vector=float(dur_b.mean() * 1e3 / 8))
      del evb
    extra["scatter_batched_1e8"] = batched_t
    log("scatter batched 1e8: %s" % batched_t)
    del data, indices, indptr, events

    # 4,000 x 4,000, 80 per row, homogeneous 0.6, 2 % events, scatter (the reference's own CPU-sized case)
    s = synth.config_event_csr_small()
    sd = {k: torch.from_numpy(v).to(dev) for k, v in s.items() if isinstance(v, np.ndarray)}
    got = bpl.event_csr_matvec(sd["data"], sd["indices"], sd["indptr"], sd["events"], shape=s["shape"], transpose=True)
    want = oracle.event_csr_matvec(s["data"], s["indices"], s["indptr"], s["events"], shape=s["shape"], transpose=True)
    if not np.array_equal(got.cpu().numpy(), want):
      raise SystemExit("parity gate failed for event_csr_matvec scatter 4,000 (homogeneous weight: bit for bit)")
    log("parity event_csr_matvec scatter 4,000           bit for bit")
    scatter_c1 = lambda: bpl.event_csr_matvec(sd["data"], sd["indices"], sd["indptr"], sd["events"],
                                              shape=s["shape"], transpose=True)
    one_c1 = single_call_us(scatter_c1)  # before any warm-up of this shape
    dur_c1, wall_c1 = time_calls(scatter_c1, args.steps, args.warmup)
    deliv = int(np.diff(s["indptr"])[s["events"]].sum())
    extra["scatter_4000"] = dict(stats(dur_c1), delivered_synapses=deliv, wall_us_per_call=wall_c1 / args.steps * 1e6,
                                 single_call_wall_us=dict(first=one_c1["first"], warm_median=one_c1["median"]))
    if not args.skip_cpu:
      t1 = time.perf_counter()
      for _ in range(2000):
        oracle.event_csr_matvec(s["data"], s["indices"], s["indptr"], s["events"], shape=s["shape"], transpose=True)
      extra["scatter_4000"]["cpu_port_1core_us"] = (time.perf_counter() - t1) / 2000 * 1e6
    # the same call through the bare C ABI with pre-marshalled arguments (what a compiled host such as XLA
    # pays per call; the figures above include this package's Python wrapper, ~15 us of argument checks)
    import ctypes
    from brainpylib_amd import _lib
    fn_raw = _lib.target("event_csr_matvec_homo_float_bool")
    out_raw = torch.empty(s["shape"][1], dtype=torch.float32, device=dev)
    bufs = (ctypes.c_void_p * 5)(*[ctypes.c_void_p(t.data_ptr()) for t in
                                   (sd["data"], sd["indices"], sd["indptr"], sd["events"], out_raw)])
    opaque = _lib.build_twouint_onebool_descriptor(s["shape"][0], s["shape"][1], True)
    stream_ptr = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    raw = lambda: fn_raw(stream_ptr, bufs, opaque, len(opaque))
    # reference point: one trivial kernel launched the same way (the launch floor of this stack)
    xs = torch.zeros(4000, device=dev)
    dur_t, wall_t = time_calls(lambda: xs.add_(1.0), 1000, 50)
    extra["scatter_4000"]["trivial_kernel_event_us"] = float(dur_t.mean() * 1e3)
    extra["scatter_4000"]["trivial_kernel_wall_us"] = wall_t / 1000 * 1e6
    dur_r, wall_r = time_calls(raw, 1000, 50)
    check(out_raw.cpu().numpy(), want, "event_csr_matvec scatter 4,000 (bare ABI)")
    extra["scatter_4000"]["bare_abi_wall_us_per_call"] = wall_r / 1000 * 1e6
    extra["scatter_4000"]["bare_abi_event_us"] = stats(dur_r)
    extra["scatter_4000"]["bare_abi_back_to_back_us"] = back_to_back_us(raw, 1000)
    extra["scatter_4000"]["wrapper_back_to_back_us"] = back_to_back_us(scatter_c1, 1000)
    extra["scatter_4000"]["trivial_kernel_back_to_back_us"] = back_to_back_us(lambda: xs.add_(1.0), 1000)
    # Its bound is the launch itself: one kernel of a few hundred nanoseconds of memory work.  Achieved = calls per
    # second back to back through the bare ABI, peak = the same for a kernel that does nothing but add 1 to 4,000 floats.
    extra["scatter_4000"]["roofline"] = roofline_record(
      "launch", 1e6 / extra["scatter_4000"]["bare_abi_back_to_back_us"],
      1e6 / extra["scatter_4000"]["trivial_kernel_back_to_back_us"], "calls/s",
      peak_measured_by="a one-launch elementwise kernel enqueued the same way in this run")
    extra["scatter_4000"]["parity"] = dict(elements=int(s["shape"][1]), outside_plain=0, violations=0, bound="bit for bit")
    # the same call replayed from a HIP graph: what a simulation loop that captures its time step pays
    gs = torch.cuda.Stream()
    gs.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(gs):
      bpl.event_csr_matvec(sd["data"], sd["indices"], sd["indptr"], sd["events"], shape=s["shape"], transpose=True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=gs):
      g_out = bpl.event_csr_matvec(sd["data"], sd["indices"], sd["indptr"], sd["events"], shape=s["shape"], transpose=True)
    graph.replay()
    torch.cuda.synchronize()
    check(g_out.cpu().numpy(), want, "event_csr_matvec scatter 4,000 (graph)")
    dur_g, wall_g = time_calls(graph.replay, args.steps, args.warmup)
    extra["scatter_4000"]["graph_replay_us"] = stats(dur_g)
    extra["scatter_4000"]["graph_replay_wall_us_per_call"] = wall_g / args.steps * 1e6
    log("scatter 4000: %s" % extra["scatter_4000"])

    # csr_matvec, 1,000,000 x 1,000,000, ~1e8 nnz
    t0 = time.time()
    m = synth.config_csr_matvec()
    log("generated csr_matvec workload in %.1f s" % (time.time() - t0))
    md = {k: torch.from_numpy(v).to(dev) for k, v in m.items() if isinstance(v, np.ndarray)}
    nnz3 = int(m["indices"].shape[0])
    oracle.set_threads(cores)
    t1 = time.perf_counter()
    want = oracle.csr_matvec(m["data"], m["indices"], m["indptr"], m["vector"], shape=m["shape"])
    t_cpu3 = time.perf_counter() - t1
    got = bpl.csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"], shape=m["shape"]).cpu().numpy()
    outside_c3 = check(got, want, "csr_matvec 1e8 nnz")
    dur3, _ = time_calls(lambda: bpl.csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"], shape=m["shape"]),
                         max(20, args.steps // 4), 5)
    bytes3 = 4 * (m["shape"][0] + 1) + 8 * nnz3 + 4 * m["shape"][1] + 4 * m["shape"][0]
    extra["csr_matvec_1e8"] = dict(stats(dur3), nnz=nnz3, gsop_per_s=nnz3 / (dur3.mean() * 1e-3) / 1e9,
                                   algorithmic_gb_per_s=bytes3 / (dur3.mean() * 1e-3) / 1e9,
                                   cpu_port_allcores_ms=t_cpu3 * 1e3, cpu_cores=cores,
                                   parity=parity_record(got, outside_c3, "rel 1e-5 / abs 1e-6"))
    # Its bound: the rate at which 4-byte elements of a 4 MB vector can be gathered from L2 at all, measured
    # here by a flat kernel over the same index and weight streams (no rows, no reduction, no output).
    ceil_rows = gather_ceiling(bench_lib, dev, md["vector"], md["indices"], md["data"], 10)
    want_sum = float(np.dot(m["vector"][m["indices"]].astype(np.float64), m["data"].astype(np.float64)))
    for r in ceil_rows:
      if abs(r["checksum"] - want_sum) > 1e-4 * abs(want_sum) + 1.0:
        raise SystemExit("flat gather kernel computed %r, expected %r" % (r["checksum"], want_sum))
    ceiling = max(r["g_gathers_per_s"] for r in ceil_rows)
    extra["csr_matvec_1e8"]["roofline"] = dict(
      bound="l2-gather", unit="G gathers/s", achieved=extra["csr_matvec_1e8"]["gsop_per_s"], peak=ceiling,
      frac=extra["csr_matvec_1e8"]["gsop_per_s"] / ceiling, peak_measured_by="bench_gather_fma, best of runs",
      runs=ceil_rows, hbm_frac=bytes3 / (dur3.mean() * 1e-3) / 1e9 / HBM_PEAK_GBS)
    log("csr_matvec 1e8: %s" % extra["csr_matvec_1e8"])
    want = oracle.csr_matvec(m["data"], m["indices"], m["indptr"], m["vector"], shape=m["shape"], transpose=True)
    mag = oracle.csr_matvec(m["data"], m["indices"], m["indptr"], np.abs(m["vector"]), shape=m["shape"], transpose=True)
    got = bpl.cusparse_csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"], shape=m["shape"],
                                  transpose=True).cpu().numpy()
    outside_c3t = check(got, want, "csr_matvec transposed 1e8 nnz", mag)
    dur3t, _ = time_calls(lambda: bpl.cusparse_csr_matvec(md["data"], md["indices"], md["indptr"], md["vector"],
                                                          shape=m["shape"], transpose=True), max(20, args.steps // 4), 5)
    extra["csr_matvec_transposed_1e8"] = dict(stats(dur3t), gsop_per_s=nnz3 / (dur3t.mean() * 1e-3) / 1e9,
                                              algorithmic_gb_per_s=bytes3 / (dur3t.mean() * 1e-3) / 1e9,
                                              parity=parity_record(got, outside_c3t,
                                                                   "rel 1e-5 / abs 1e-6 + 4 eps sum|addends|"))
    # the sorted scatter writes and reads every (16-bit column in its window, product) pair once more: 8 + 12
    # bytes per nonzero
    extra["csr_matvec_transposed_1e8"]["roofline"] = dict(
      bound="hbm", unit="GB/s", achieved=bytes3 / (dur3t.mean() * 1e-3) / 1e9, peak=HBM_PEAK_GBS,
      frac=bytes3 / (dur3t.mean() * 1e-3) / 1e9 / HBM_PEAK_GBS,
      bytes_moved_by_design_gb_per_s=(bytes3 + 12.0 * nnz3) / (dur3t.mean() * 1e-3) / 1e9)
    log("csr_matvec transposed 1e8: %s" % extra["csr_matvec_transposed_1e8"])
    # a dense vector short enough for LDS (up to 159 KB): 200,000 x 19,000, 100 per row, 2.0e7 nnz
    rng_s = np.random.default_rng(23)
    ix_s, ip_s = synth.counted_csr(np.full(200_000, 100), 19_000, seed=23)
    d_s = rng_s.random(ix_s.shape[0], dtype=np.float32)
    v_s = rng_s.standard_normal(19_000).astype(np.float32)
    dev_s = [torch.from_numpy(a_).to(dev) for a_ in (d_s, ix_s, ip_s, v_s)]
    got = bpl.csr_matvec(*dev_s, shape=(200_000, 19_000)).cpu().numpy()
    check(got, oracle.csr_matvec(d_s, ix_s, ip_s, v_s, shape=(200_000, 19_000)), "csr_matvec vector in LDS")
    dur_s, _ = time_calls(lambda: bpl.csr_matvec(*dev_s, shape=(200_000, 19_000)), max(20, args.steps // 4), 5)
    extra["csr_matvec_2e7_vector_in_lds"] = dict(stats(dur_s), gsop_per_s=ix_s.shape[0] / (dur_s.mean() * 1e-3) / 1e9,
                                                 algorithmic_gb_per_s=8.0 * ix_s.shape[0] / (dur_s.mean() * 1e-3) / 1e9)
    log("csr_matvec 2e7, vector in LDS: %s" % extra["csr_matvec_2e7_vector_in_lds"])
    # the same matrix transposed: the output (19,000 columns) fits two float64 windows in LDS; and 1,000,000 x 16,000
    # with 50 per row, whose output fits one (every workgroup walks an equal share of the nonzeros into its window)
    u_s = rng_s.standard_normal(200_000).astype(np.float32)
    u_dev = torch.from_numpy(u_s).to(dev)
    got = bpl.cusparse_csr_matvec(dev_s[0], dev_s[1], dev_s[2], u_dev, shape=(200_000, 19_000), transpose=True).cpu().numpy()
    check(got, oracle.csr_matvec(d_s, ix_s, ip_s, u_s, shape=(200_000, 19_000), transpose=True),
          "csr_matvec transposed, two LDS windows",
          oracle.csr_matvec(d_s, ix_s, ip_s, np.abs(u_s), shape=(200_000, 19_000), transpose=True))
    ix_n, ip_n = synth.counted_csr(np.full(1_000_000, 50), 16_000, seed=29)
    d_n = rng_s.random(ix_n.shape[0], dtype=np.float32)
    u_n = rng_s.standard_normal(1_000_000).astype(np.float32)
    dev_n = [torch.from_numpy(a_).to(dev) for a_ in (d_n, ix_n, ip_n, u_n)]
    got = bpl.cusparse_csr_matvec(*dev_n, shape=(1_000_000, 16_000), transpose=True).cpu().numpy()
    check(got, oracle.csr_matvec(d_n, ix_n, ip_n, u_n, shape=(1_000_000, 16_000), transpose=True),
          "csr_matvec transposed, one LDS window",
          oracle.csr_matvec(d_n, ix_n, ip_n, np.abs(u_n), shape=(1_000_000, 16_000), transpose=True))
    dur_n, _ = time_calls(lambda: bpl.cusparse_csr_matvec(*dev_n, shape=(1_000_000, 16_000), transpose=True),
                          max(20, args.steps // 4), 5)
    bytes_n = 8.0 * ix_n.shape[0] + 4.0 * (1_000_001 + 1_000_000 + 16_000)
    extra["csr_matvec_transposed_5e7_output_in_lds"] = dict(
      stats(dur_n), gsop_per_s=ix_n.shape[0] / (dur_n.mean() * 1e-3) / 1e9,
      roofline=dict(bound="hbm", unit="GB/s", achieved=bytes_n / (dur_n.mean() * 1e-3) / 1e9, peak=HBM_PEAK_GBS,
                    frac=bytes_n / (dur_n.mean() * 1e-3) / 1e9 / HBM_PEAK_GBS))
    log("csr_matvec transposed 5e7, output in LDS: %s" % extra["csr_matvec_transposed_5e7_output_in_lds"])
    del dev_n, ix_n, ip_n, d_n, u_n
    del dev_s
    # the same 1,000,000 x 1,000,000 matrix (100 nonzeros per row) driven by events, 1 % and 5 % of
    # the rows active: the shape of a million-neuron network's synaptic update (output far wider than LDS)
    wide = {}
    for rate in (0.01, 0.05):
      ev_np = np.random.default_rng(17).random(m["shape"][0]) < rate
      ev_w = torch.from_numpy(ev_np).to(dev)
      want = oracle.event_csr_matvec(m["data"], m["indices"], m["indptr"], ev_np, shape=m["shape"], transpose=True)
      mag = oracle.event_csr_matvec(np.abs(m["data"]), m["indices"], m["indptr"], ev_np, shape=m["shape"], transpose=True)
      got = bpl.event_csr_matvec(md["data"], md["indices"], md["indptr"], ev_w, shape=m["shape"], transpose=True)
      check(got.cpu().numpy(), want, "event_csr_matvec scatter 1e6 x 1e6 at %g" % rate, mag)
      dur_w, _ = time_calls(lambda: bpl.event_csr_matvec(md["data"], md["indices"], md["indptr"], ev_w, shape=m["shape"],
                                                         transpose=True), args.steps, 5)
      delivered = int(np.diff(m["indptr"])[ev_np].sum())
      wide["events_%g" % rate] = dict(stats(dur_w), delivered_synapses=delivered,
                                      gsop_per_s=delivered / (dur_w.mean() * 1e-3) / 1e9)
    extra["scatter_1e6x1e6_100_per_row"] = wide
    log("event scatter 1e6 x 1e6: %s" % wide)
    # the gather over the same matrix (5 % of the columns have an event), and over 500,000 x 500,000 with 100 per
    # row: short rows behind a bitmap of 125 KB (one workgroup per CU) and of 62.5 KB (two): the walks over
    # the nonzeros that look rows up for the hits only
    short = {}
    for tag, sm, smd in (("1e6x1e6", m, md), ("5e5x5e5", None, None)):
      if sm is None:
        r_s = np.random.default_rng(31)
        sm = dict(shape=(500_000, 500_000), indices=r_s.integers(0, 500_000, size=50_000_000, dtype=np.int32),
                  indptr=(np.arange(500_001, dtype=np.int64) * 100).astype(np.int32),
                  data=r_s.random(50_000_000, dtype=np.float32))
        smd = {k: torch.from_numpy(v).to(dev) for k, v in sm.items() if isinstance(v, np.ndarray)}
      ev_np = np.random.default_rng(18).random(sm["shape"][1]) < 0.05
      ev_s = torch.from_numpy(ev_np).to(dev)
      nnz_s = int(sm["indices"].shape[0])
      for name, w_np, w_dev in (("heter", sm["data"], smd["data"]),
                                ("homo", sm["data"][:1], smd["data"][:1].contiguous())):
        want = oracle.event_csr_matvec(w_np, sm["indices"], sm["indptr"], ev_np, shape=sm["shape"])
        mag = oracle.event_csr_matvec(np.abs(w_np), sm["indices"], sm["indptr"], ev_np, shape=sm["shape"])
        got = bpl.event_csr_matvec(w_dev, smd["indices"], smd["indptr"], ev_s, shape=sm["shape"])
        check(got.cpu().numpy(), want, "event_csr_matvec gather %s %s" % (tag, name), mag)
        dur_s, _ = time_calls(lambda: bpl.event_csr_matvec(w_dev, smd["indices"], smd["indptr"], ev_s, shape=sm["shape"]),
                              args.steps, 5)
        bytes_s = nnz_s * (8 if name == "heter" else 4) + 8 * sm["shape"][0]
        short["%s_%s" % (tag, name)] = dict(
          stats(dur_s), nnz=nnz_s,
          roofline=dict(bound="hbm", unit="GB/s", achieved=bytes_s / (dur_s.mean() * 1e-3) / 1e9, peak=HBM_PEAK_GBS,
                        frac=bytes_s / (dur_s.mean() * 1e-3) / 1e9 / HBM_PEAK_GBS))
      if tag != "1e6x1e6":
        del sm, smd
    extra["gather_100_per_row"] = short
    log("event gather, 100 per row: %s" % short)
    # a mid-size projection, 32,000 x 8,192 with about 1,000 nonzeros per row: the walk into LDS windows whose
    # workgroups find the active rows themselves, at three activities
    counts_m = np.maximum(1, np.random.default_rng(23).poisson(1000, 32_000))
    ix_m, ip_m = synth.counted_csr(counts_m, 8192, seed=5)
    d_m = np.random.default_rng(24).random(ix_m.shape[0], dtype=np.float32)
    dev_m = [torch.from_numpy(a).to(dev) for a in (d_m, ix_m, ip_m)]
    mid = {}
    for rate in (0.01, 0.05, 0.2):
      ev_np = np.random.default_rng(25).random(32_000) < rate
      ev_m = torch.from_numpy(ev_np).to(dev)
      want = oracle.event_csr_matvec(d_m, ix_m, ip_m, ev_np, shape=(32_000, 8192), transpose=True)
      mag = oracle.event_csr_matvec(np.abs(d_m), ix_m, ip_m, ev_np, shape=(32_000, 8192), transpose=True)
      got = bpl.event_csr_matvec(*dev_m, ev_m, shape=(32_000, 8192), transpose=True)
      check(got.cpu().numpy(), want, "event_csr_matvec scatter 32,000 x 8,192 at %g" % rate, mag)
      dur_m, _ = time_calls(lambda: bpl.event_csr_matvec(*dev_m, ev_m, shape=(32_000, 8192), transpose=True), args.steps, 5)
      delivered = int(np.diff(ip_m)[ev_np].sum())
      mid["events_%g" % rate] = dict(stats(dur_m), delivered_synapses=delivered,
                                     gsop_per_s=delivered / (dur_m.mean() * 1e-3) / 1e9)
    extra["scatter_32000x8192_1000_per_row"] = mid
    log("event scatter 32,000 x 8,192: %s" % mid)
    del dev_m

  if not args.skip_extra:
    del md
    torch.cuda.empty_cache()
    # jitconn event matvec: 1e6 x 1e6 implicit matrix, conn_prob 0.001, events 1 %, seed 42
    j = synth.config_jitconn_event()
    n = j["shape"][0]
    ev = torch.from_numpy(j["events"]).to(dev)
    # number of implicit synapses the generator produces (exact): sum of a homo matvec over ones
    ones = torch.ones(n, dtype=torch.float64, device=dev)
    generated = int(bpl.matvec_prob_conn_homo_weight(ones, 1.0, conn_prob=j["conn_prob"], shape=j["shape"],
                                                     seed=j["seed"]).sum().item())
    lp = oracle.log_p_of(j["conn_prob"])
    out_row = bpl.event_matvec_prob_conn_homo_weight(ev, j["weight"], conn_prob=j["conn_prob"], shape=j["shape"],
                                                     seed=j["seed"]).cpu().numpy()
    for r in np.random.default_rng(0).choice(n, 64, replace=False):
      idx, _ = oracle.jitconn_stream_indices(j["seed"] + int(r), lp, n)
      if out_row[r] != np.float32(j["events"][idx].sum()) * np.float32(0.1):
        raise SystemExit("parity gate failed for jitconn event matvec row %d" % r)
    jit = {"generated_synapses": generated,
           "parity_row_walk": dict(elements=64, outside_plain=0, violations=0,
                                   bound="bit for bit (64 sampled rows against single-stream oracle walks)")}
    # column walk: the whole output against the oracle's streams of the active columns (counts: exact)
    out_col = bpl.event_matvec_prob_conn_homo_weight(ev, 1.0, conn_prob=j["conn_prob"], shape=j["shape"], seed=j["seed"],
                                                     outdim_parallel=False).cpu().numpy()
    want_col = np.zeros(n)
    pairs = 0
    for col in np.flatnonzero(j["events"]):
      idx, _ = oracle.jitconn_stream_indices(j["seed"] + int(col), lp, n)
      np.add.at(want_col, idx, 1.0)
      pairs += idx.shape[0]
    if not np.array_equal(out_col.astype(np.float64), want_col):
      raise SystemExit("parity gate failed for the jitconn column walk (whole output, counts)")
    log("parity jitconn column walk 1e6 x 1e6        whole output bit for bit (%d pairs)" % pairs)
    jit["parity_column_walk"] = dict(elements=n, outside_plain=0, violations=0, bound="bit for bit (whole output)")
    jit["column_walk_pairs"] = pairs
    # the row walk is bound by VALU issue: peak = CUs x 64 lanes x clock lane-instructions per second (one
    # wave64 instruction per SIMD every four cycles).  The number of vector instructions a call executes is a
    # counter reading (SQ_INSTS_VALU, rocprofv3 --pmc run of this workload, `--pmc jitconn`), since counters
    # cannot be read in-process; the time it is divided by is measured here.
    props = torch.cuda.get_device_properties(dev)
    clock_hz = float(getattr(props, "clock_rate", 2400000)) * 1e3
    jit["valu_roofline"] = {"bound": "valu", "peak_lane_instr_per_s": props.multi_processor_count * 64 * clock_hz,
                            "compute_units": props.multi_processor_count, "clock_ghz": clock_hz / 1e9}
    for transpose in (False, True):
      for odp in (True, False):
        fn = lambda: bpl.event_matvec_prob_conn_homo_weight(ev, j["weight"], conn_prob=j["conn_prob"], shape=j["shape"],
                                                            seed=j["seed"], transpose=transpose, outdim_parallel=odp)
        d, _ = time_calls(fn, max(10, args.steps // 10), 3)
        key = "transpose=%s,outdim_parallel=%s" % (transpose, odp)
        jit[key] = dict(stats(d), implicit_gsyn_per_s=generated / (d.mean() * 1e-3) / 1e9)
    call_us = jit["transpose=False,outdim_parallel=True"]["mean_us"]
    rec_j = recorded_counters("jitconn_rowwalk_1e9", call_us, generated_synapses=generated)
    vr = jit["valu_roofline"]
    if rec_j:
      lane_instr = rec_j["valu_wave_instr_per_call"] * 64.0
      jit["roofline_row_walk"] = roofline_record(
        "valu", lane_instr / (call_us * 1e-6) / 1e12, vr["peak_lane_instr_per_s"] / 1e12, "T lane instructions/s",
        instruction_count_recorded_in=rec_j["profile"])
      vr.update(achieved_lane_instr_per_s=lane_instr / (call_us * 1e-6),
                frac=lane_instr / (call_us * 1e-6) / vr["peak_lane_instr_per_s"],
                valu_instr_per_64_synapses_recorded=rec_j["valu_instr_per_64_synapses"],
                valu_active_over_simd_cycles_recorded=rec_j["valu_active_over_simd_cycles"],
                recorded_in=rec_j["profile"],
                recorded_at=dict(git_rev=rec_j["git_rev"], kernel=rec_j["kernel"], call_us=rec_j["kernel_us"]))
    else:
      vr.update(achieved_lane_instr_per_s=None, frac=None, recorded_in=None)
    if not args.skip_cpu:
      # reference CPU algorithm (one sequential mt19937) on the first 4,000 rows of the same matrix
      rows = 4000
      t1 = time.perf_counter()
      oracle.jitconn_matvec(j["events"], log_p=lp, seed=j["seed"], n_row=rows, n_col=n, per_stream_seed=False)
      t_cpu = time.perf_counter() - t1
      jit["cpu_port_1core"] = {"implicit_gsyn_per_s": generated * (rows / n) / t_cpu / 1e9,
                               "sample": "first %d of %d rows, %.2f s" % (rows, n, t_cpu)}
    # dense-vector twin (jitconn matvec): same streams, float inputs gathered from L2
    vec = torch.randn(n, dtype=torch.float32, device=dev)
    for odp in (True, False):
      fn = lambda: bpl.matvec_prob_conn_homo_weight(vec, j["weight"], conn_prob=j["conn_prob"], shape=j["shape"],
                                                    seed=j["seed"], outdim_parallel=odp)
      d, _ = time_calls(fn, max(5, args.steps // 20), 2)
      # every synapse gathers one element of the 4 MB vector from the L2 (row walk) or adds one pair through the bins
      # (column walk): set beside the flat-gather ceiling of this run, measured over the csr_matvec arrays above
      jit["dense_matvec,outdim_parallel=%s" % odp] = dict(
        stats(d), implicit_gsyn_per_s=generated / (d.mean() * 1e-3) / 1e9,
        roofline=roofline_record("l2-gather" if odp else "l2-gather (pairs through bins)",
                                 generated / (d.mean() * 1e-3) / 1e9, ceiling, "G synapses/s",
                                 peak_measured_by="bench_gather_fma over 1e8 nonzeros and a 1,000,000-element vector"))
    # parity of the dense walks at full size: a 0/1 vector gives counts, which are exact in any order: the row walk
    # against the event walk's counts (64 sampled rows checked above), the column walk against the event column walk
    vec01 = ev.to(torch.float32)
    for odp, want_01 in ((True, out_row / np.float32(0.1)), (False, out_col)):
      got_01 = bpl.matvec_prob_conn_homo_weight(vec01, 1.0, conn_prob=j["conn_prob"], shape=j["shape"], seed=j["seed"],
                                                outdim_parallel=odp).cpu().numpy()
      if not np.array_equal(got_01, np.rint(want_01).astype(np.float32)):
        raise SystemExit("parity gate failed for the dense jitconn walk (outdim_parallel=%s) on a 0/1 vector" % odp)
      jit["dense_matvec,outdim_parallel=%s" % odp]["parity"] = dict(
        elements=n, outside_plain=0, violations=0, bound="bit for bit (0/1 vector: counts equal the event walk's)")
    log("parity dense jitconn walks 1e6 x 1e6        0/1 vector: whole outputs equal the event walks' counts")
    # the event column walk: three short kernels (list, seed, walk) and the sum of the bins; its traffic by design is
    # the pairs written and read once (8 bytes each way) plus the output
    cw = jit["transpose=False,outdim_parallel=False"]
    cw["roofline"] = roofline_record("hbm", (16.0 * pairs + 4.0 * n + n) / (cw["mean_us"] * 1e-6) / 1e9, HBM_PEAK_GBS,
                                     "GB/s", note="bytes the design moves (pairs written and read once); the chain of "
                                                  "launches and the serial stream walk bound it, not the memory")
    extra["jitconn_event_matvec_1e9"] = jit
    log("jitconn event matvec: %s" % jit)

    # jitconn matmat: 10,000 x 10,000, conn_prob 0.1, N(0, 0.01^2), times B[10000, 128]
    mm = synth.config_jitconn_matmat()
    X = torch.from_numpy(np.ascontiguousarray(mm["B"].T)).to(dev)
    fn = lambda: bpl.matmat_prob_conn_normal_weight(X, w_mu=mm["w_mu"], w_sigma=mm["w_sigma"], conn_prob=mm["conn_prob"],
                                                    shape=mm["shape"], seed=mm["seed"])
    got = fn().cpu().numpy()
    lp = oracle.log_p_of(mm["conn_prob"])
    # the oracle over all 128 rows of X (every stream generated once and applied to every row), with
    # sum(|w x|) per output for the reordering term; single-threaded it is also the CPU figure of this leg
    oracle.set_threads(1)
    t1 = time.perf_counter()
    want, mag = oracle.jitconn_matmat(np.ascontiguousarray(mm["B"].T), w_kind="normal", w_a=mm["w_mu"], w_b=mm["w_sigma"],
                                      log_p=lp, seed=mm["seed"], n=mm["shape"][1], return_abs=True)
    t_cpu = time.perf_counter() - t1
    outside_mm = check(got, want, "jitconn matmat 10,000 x 10,000 x 128", mag)
    gen_mm = int(bpl.matvec_prob_conn_homo_weight(torch.ones(mm["shape"][0], dtype=torch.float64, device=dev), 1.0,
                                                  conn_prob=mm["conn_prob"], shape=mm["shape"], seed=mm["seed"],
                                                  transpose=True).sum().item())
    d, _ = time_calls(fn, max(10, args.steps // 10), 3)
    extra["jitconn_matmat_1e4x128"] = dict(stats(d), generated_synapses=gen_mm,
                                           gfma_per_s=gen_mm * 128 / (d.mean() * 1e-3) / 1e9,
                                           l2_gather_gb_per_s=gen_mm * 128 * 4 / (d.mean() * 1e-3) / 1e9,
                                           parity=dict(elements=int(got.size), outside_plain=outside_mm, violations=0),
                                           cpu_port_1core_s_per_call=t_cpu,
                                           cpu_sample="one full call, every stream generated once (%.2f s)" % t_cpu)
    mm_leg = extra["jitconn_matmat_1e4x128"]
    rec_m = recorded_counters("jitconn_matmat_1e4x128", mm_leg["mean_us"], generated_synapses=gen_mm)
    if rec_m:
      # instruction issue: vector instructions per call (SQ_INSTS_VALU of the recorded --pmc matmat run) x 64 lanes
      # over this run's time, against CUs x 64 lanes x clock; and the 128-byte requests its loads send to the L2s
      lane_instr = rec_m["valu_wave_instr_per_call"] * 64.0
      mm_leg["roofline"] = roofline_record(
        "valu", lane_instr / (mm_leg["mean_us"] * 1e-6) / 1e12, vr["peak_lane_instr_per_s"] / 1e12,
        "T lane instructions/s", instruction_count_recorded_in=rec_m["profile"],
        valu_instr_per_synapse_recorded=rec_m["valu_wave_instr_per_call"] / gen_mm,
        l2_read_tb_per_s=rec_m["l2_read_requests_per_call"] * 128.0 / (mm_leg["mean_us"] * 1e-6) / 1e12,
        recorded_at=dict(git_rev=rec_m["git_rev"], kernel=rec_m["kernel"], call_us=rec_m["kernel_us"]))
    else:
      mm_leg["roofline"] = None
    # the same call while the clocks are still low: the first calls after an idle second
    time.sleep(1.0)
    d_cold, _ = time_calls(fn, 10, 0, warm_s=0.0)
    mm_leg["first_10_calls_after_1s_idle_us"] = stats(d_cold)
    log("jitconn matmat: %s" % extra["jitconn_matmat_1e4x128"])

    # ---------------------------------------------------------------------------------------------
    # event_info: 1,000 event vectors of 100,000 bool events, density 0.1 (the shape of the
    # reference's event_info_VS_jax_operators.py, whose docstring reports 2.78 ms per call on its GPU)
    # ---------------------------------------------------------------------------------------------
    ev_np = np.random.default_rng(11).random((1000, 100_000)) < 0.1
    ev_t = torch.from_numpy(ev_np).to(dev)
    ids, num = bpl.event_info(ev_t)
    w_ids, w_num = oracle.event_info(ev_np[17])
    ok = bool(np.array_equal(ids[17].cpu().numpy(), w_ids)) and int(num[17]) == int(w_num[0]) and \
        bool(np.array_equal(num.cpu().numpy(), ev_np.sum(axis=1)))
    log("parity event_info (1000, 100000)          row 17 and all counts exact: %s" % ok)
    if not ok:
      raise SystemExit("event_info parity failed")
    d_ei, _ = time_calls(lambda: bpl.event_info(ev_t), max(10, args.steps // 10), 3)
    extra["event_info_1000x100000"] = dict(stats(d_ei), gb_per_s=(ev_np.size * 5 + 4000) / (d_ei.mean() * 1e-3) / 1e9,
                                           reference_docstring_ms=2.782)
    log("event_info: %s" % extra["event_info_1000x100000"])
    del ev_t, ids, num

  # One flat record per configuration of the benchmark's list (C1 ... C5, T = the transposed / scatter / column
  # orientation): microseconds per call, fraction of the leg's own roofline, elements outside the plain parity
  # bound.  Scalars only, inside "roofline", and once more as the last lines on stderr, so that they are on record
  # wherever the line or the end of the log is kept.
  flat, tags = {}, []
  if not args.skip_extra:
    def put(tag, leg, roof=None, par=None):
      tags.append(tag)
      roof = leg.get("roofline") if roof is None else roof
      par = leg.get("parity") if par is None else par
      flat[tag + "_us"] = round(leg["mean_us"], 2)
      if roof:
        flat[tag + "_bound"] = roof["bound"]
        flat[tag + "_frac"] = round(roof["frac"], 4)
      if par:
        flat[tag + "_outside_plain"] = "%d/%d" % (par["outside_plain"], par["elements"])
    jit = extra["jitconn_event_matvec_1e9"]
    put("C1_scatter_4000", dict(extra["scatter_4000"], mean_us=extra["scatter_4000"]["bare_abi_back_to_back_us"]))
    put("C2_gather_homo", extra["gather_homo_1e8"])
    put("C2T_scatter", extra["scatter_1e8"])
    put("C3_csr_matvec", extra["csr_matvec_1e8"])
    put("C3T_csr_matvec", extra["csr_matvec_transposed_1e8"])
    put("C4_row_walk", jit["transpose=False,outdim_parallel=True"], jit.get("roofline_row_walk"), jit["parity_row_walk"])
    put("C4_column_walk", jit["transpose=False,outdim_parallel=False"], None, jit["parity_column_walk"])
    put("C4_dense_row_walk", jit["dense_matvec,outdim_parallel=True"])
    put("C4_dense_column_walk", jit["dense_matvec,outdim_parallel=False"])
    put("C5_matmat", extra["jitconn_matmat_1e4x128"])
  log("summary C2 gather (headline): %.1f us kernel, %.1f us wall per step, hbm frac %.3f, outside plain %d/%d" % (
    kernel_ms * 1e3, ms_per_step * 1e3, achieved / HBM_PEAK_GBS, outside_g, got_g.size))
  for tag in tags:
    log("summary %-22s %9.1f us  %-28s frac %-7s outside plain %s" % (
      tag, flat[tag + "_us"], flat.get(tag + "_bound", "-"), flat.get(tag + "_frac", "-"),
      flat.get(tag + "_outside_plain", "-")))

  result = {
    "metric": "GSOP/s + % HBM roofline, event_csr_matvec 1e8 nnz; jitconn GSOP/s at p=0.001",
    "value": value,
    "unit": "GSOP/s (CSR nonzeros scanned per second, event_csr_matvec transpose=False)",
    "n_gpus": 1,
    "steps": args.steps,
    "warmup": args.warmup,
    "ms_per_step": ms_per_step,
    "higher_is_better": True,
    "scaling": "weak",
    "vs_baseline": None,
    "dtype": "f32",
    "data": "synthetic",
    "config": {"workload": "event_csr_matvec heterogeneous 100000x100000, nnz~Binomial(1e5,0.01)/row (%d nnz), "
                           "weights N(0,0.1^2), events Bernoulli(0.05), transpose=False, seed 1" % nnz},
    # traffic: HBM bytes per launch of this kernel on this workload, from two rocprofv3 --pmc runs (FETCH_SIZE,
    # WRITE_SIZE; `--pmc gather` mode above) scaled by what a 400 MB copy reads on the same counters; counters
    # cannot be read in-process, so the figure is the one recorded in profiles/recorded_counters.json, emitted
    # only while this run's kernel time agrees with the time at which it was recorded (else null)
    "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                 "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                 "traffic_recorded_in": rec["profile"] if rec else None,
                 "traffic_recorded_at": dict(git_rev=rec["git_rev"], kernel=rec["kernel"],
                                             kernel_us=rec["kernel_us"]) if rec else None,
                 "kernel": "csr_gather_kernel<float,bool,heter,event,lds-bitmap>",
                 "algorithmic_bytes_per_launch": bytes_gather, "kernel_us": kernel_ms * 1e3,
                 # the same launch against what plain loads of its real traffic reach in this run
                 "streaming_ceiling_gb_per_s": stream_rate,
                 "frac_of_streaming_ceiling": (traffic / (kernel_ms * 1e-3) / 1e9 / stream_rate) if traffic else None,
                 "outside_plain_parity_bound": "%d/%d" % (outside_g, got_g.size),
                 "clock_warm_s_before_each_timed_region": CLOCK_WARM_S,
                 **flat},
    "cpu_baseline": cpu_baseline,
    "extra": extra,
  }
  print(json.dumps(result), flush=True)


if __name__ == "__main__":
  main()
