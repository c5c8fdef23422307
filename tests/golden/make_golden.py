"""Writes the golden fixtures in this directory by running the reference's own CPU kernels
(lib/cpu_jitconn_*.cpp, lib/cpu_event_sum.cc, lib/cpu_atomic_sum.cc, lib/cpu_event_prod.cc,
lib/cpu_atomic_prod.cc), compiled unmodified by
`make -C oracle ref`.  Runs only where the reference tree is mounted; the fixtures it writes are
committed.

    python tests/golden/make_golden.py            # all fixtures
    python tests/golden/make_golden.py compat     # only compat_cpu_reference.npz
    python tests/golden/make_golden.py prod       # only compat_prod_cpu_reference.npz

jitconn_cpu_reference.npz
    the reference CPU backend as it ships: ONE sequential generator per matrix.  For every case
    `<i>`: `in_<i>` (input vector), `out_<i>` (custom-call result), `meta_<i>` (json).
jitconn_cpu_reference_streams.npz
    the same kernels run one generator stream at a time: output element (or scattered column)
    `s` is the reference's result for a one-stream matrix seeded `seed + s`.  This is the
    generator contract of the HIP kernels.
event_sum_cpu_reference.npz
    lib/cpu_event_sum.cc on seeded CSR matrices (event_csr_matvec, transpose=True, bool events).
compat_cpu_reference.npz
    lib/cpu_atomic_sum.cc (coo_atomic_sum, homogeneous and heterogeneous, 32- and 64-bit ids) and
    the 64-bit instantiation of lib/cpu_event_sum.cc, on seeded random connections.
compat_prod_cpu_reference.npz
    lib/cpu_atomic_prod.cc (coo_atomic_prod) and lib/cpu_event_prod.cc (csr_event_prod), homogeneous
    and heterogeneous, 32- and 64-bit ids, on seeded random connections with weights near 1.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from oracle import ref  # noqa: E402
import benchdata as synth  # noqa: E402

JIT_SHAPES = [(100, 200), (10, 1000), (2, 1000), (1000, 10), (1000, 2)]
PROBS = [0.01, 0.1, 0.5]
WEIGHTS = [("homo", 0.0, 0.0), ("uniform", -1.0, 2.0), ("normal", 0.5, 2.0)]
SEED = 1234


def make_input(rng, kind, n):
  if kind == "bool":
    return rng.random(n) < 0.3, None
  if kind in ("f32ev", "f64ev"):
    dt = np.float32 if kind == "f32ev" else np.float64
    return ((rng.random(n) < 0.3) * rng.random(n)).astype(dt), False
  dt = np.float32 if kind == "f32" else np.float64
  return rng.standard_normal(n).astype(dt), True


def jitconn_cases():
  rng = np.random.default_rng(2024)
  for (n_row, n_col) in JIT_SHAPES:
    for p in PROBS:
      for col_walk in (False, True):
        for (wk, a, b) in WEIGHTS:
          for kind, out_dt in (("bool", "float32"), ("bool", "float64"), ("f32ev", None),
                               ("f32", None), ("f64", None)):
            inp, dense = make_input(rng, kind, n_col)
            meta = dict(n_row=n_row, n_col=n_col, conn_prob=p, col_walk=col_walk, w_kind=wk, w_a=a, w_b=b,
                        seed=SEED, dense=dense, out_dtype=out_dt)
            yield inp, meta


def run_ref(inp, meta, *, n_row=None, n_col=None, seed=None, sub=None):
  return ref.jitconn_matvec(
    inp if sub is None else sub, w_kind=meta["w_kind"], w_a=meta["w_a"], w_b=meta["w_b"],
    log_p=oracle.log_p_of(meta["conn_prob"]), seed=meta["seed"] if seed is None else seed,
    n_row=meta["n_row"] if n_row is None else n_row, n_col=meta["n_col"] if n_col is None else n_col,
    col_walk=meta["col_walk"], out_dtype=np.dtype(meta["out_dtype"]) if meta["out_dtype"] else None,
    dense=meta["dense"])


def compat_fixture():
  out = {}
  i = 0
  for pre, post, conn in [(200, 200, 20000), (50, 300, 4000), (300, 7, 5000), (1, 1, 10)]:
    for homo in (True, False):
      for dt in (np.float32, np.float64):
        for wide in (False, True):
          rng = np.random.default_rng(900 + i)
          pre_ids = rng.integers(0, pre, size=conn).astype(np.int64 if wide else np.int32)
          post_ids = rng.integers(0, post, size=conn).astype(np.int64 if wide else np.int32)
          values = np.array([0.37], dtype=dt) if homo else rng.standard_normal(pre).astype(dt)
          out["as_values_%d" % i], out["as_pre_%d" % i], out["as_post_%d" % i] = values, pre_ids, post_ids
          out["as_num_%d" % i] = np.array(post)
          out["as_out_%d" % i] = ref.coo_atomic_sum(values, post_ids, post, None if homo else pre_ids, wide=wide)
          i += 1
  j = 0
  for shape in [(100, 200), (1000, 10), (2, 10000)]:
    for homo in (True, False):
      for dt in (np.float32, np.float64):
        indices, indptr = synth.bernoulli_csr(shape[0], shape[1], 0.4, seed=300 + j)
        rng = np.random.default_rng(700 + j)
        data = np.array([1.5], dtype=dt) if homo else rng.standard_normal(indices.shape[0]).astype(dt)
        events = rng.random(shape[0]) < 0.2
        out["es_data_%d" % j], out["es_events_%d" % j], out["es_shape_%d" % j] = data, events, np.array(shape)
        out["es_indices_%d" % j], out["es_indptr_%d" % j] = indices.astype(np.int64), indptr.astype(np.int64)
        out["es_out_%d" % j] = ref.csr_event_sum(data, indices, indptr, events, shape=shape, wide=True)
        j += 1
  np.savez_compressed(os.path.join(HERE, "compat_cpu_reference.npz"), **out)
  print("wrote", i, "coo_atomic_sum cases and", j, "64-bit csr_event_sum cases")


def prod_fixture():
  out = {}
  i = 0
  # weights near 1 keep products of a few hundred factors inside the normal range
  for pre, post, conn in [(200, 200, 4000), (50, 300, 2000), (300, 7, 600), (1, 1, 10)]:
    for homo in (True, False):
      for dt in (np.float32, np.float64):
        for wide in (False, True):
          rng = np.random.default_rng(1900 + i)
          pre_ids = rng.integers(0, pre, size=conn).astype(np.int64 if wide else np.int32)
          post_ids = rng.integers(0, post, size=conn).astype(np.int64 if wide else np.int32)
          values = np.array([0.97], dtype=dt) if homo else rng.uniform(0.9, 1.1, pre).astype(dt)
          if not homo and i % 4 == 1:
            values[rng.integers(0, pre, 3)] *= -1  # signs
          out["ap_values_%d" % i], out["ap_pre_%d" % i], out["ap_post_%d" % i] = values, pre_ids, post_ids
          out["ap_num_%d" % i] = np.array(post)
          out["ap_out_%d" % i] = ref.coo_atomic_prod(values, post_ids, post, None if homo else pre_ids, wide=wide)
          i += 1
  j = 0
  for shape in [(100, 200), (300, 10), (2, 3000)]:
    for homo in (True, False):
      for dt in (np.float32, np.float64):
        for wide in (False, True):
          indices, indptr = synth.bernoulli_csr(shape[0], shape[1], 0.3, seed=1300 + j)
          rng = np.random.default_rng(1700 + j)
          data = np.array([1.03], dtype=dt) if homo else rng.uniform(0.9, 1.1, indices.shape[0]).astype(dt)
          events = rng.random(shape[0]) < 0.3
          it = np.int64 if wide else np.int32
          out["ep_data_%d" % j], out["ep_events_%d" % j], out["ep_shape_%d" % j] = data, events, np.array(shape)
          out["ep_indices_%d" % j], out["ep_indptr_%d" % j] = indices.astype(it), indptr.astype(it)
          out["ep_out_%d" % j] = ref.csr_event_prod(data, indices, indptr, events, shape=shape, wide=wide)
          j += 1
  np.savez_compressed(os.path.join(HERE, "compat_prod_cpu_reference.npz"), **out)
  print("wrote", i, "coo_atomic_prod cases and", j, "csr_event_prod cases")


def main():
  if len(sys.argv) > 1 and sys.argv[1] == "prod":
    prod_fixture()
    return
  compat_fixture()
  if len(sys.argv) > 1 and sys.argv[1] == "compat":
    return
  assert ref.available(), "run `make -C oracle ref` first"
  seq, streams = {}, {}
  for i, (inp, meta) in enumerate(jitconn_cases()):
    seq["in_%d" % i] = inp
    seq["meta_%d" % i] = np.array(json.dumps(meta))
    seq["out_%d" % i] = run_ref(inp, meta)
    # one stream at a time
    if meta["col_walk"]:
      acc = None
      for c in range(meta["n_col"]):
        part = run_ref(inp, meta, n_col=1, seed=meta["seed"] + c, sub=inp[c:c + 1])
        acc = part.astype(np.float64) if acc is None else acc + part
      streams["out_%d" % i] = acc  # float64 sum of the per-column contributions
    else:
      streams["out_%d" % i] = np.concatenate(
        [run_ref(inp, meta, n_row=1, seed=meta["seed"] + r) for r in range(meta["n_row"])])
  np.savez_compressed(os.path.join(HERE, "jitconn_cpu_reference.npz"), **seq)
  np.savez_compressed(os.path.join(HERE, "jitconn_cpu_reference_streams.npz"), **streams)

  ev = {}
  i = 0
  for shape in [(100, 200), (200, 100), (10, 1000), (2, 10000), (1000, 10), (10000, 2)]:
    for homo in (True, False):
      for dt in (np.float32, np.float64):
        indices, indptr = synth.bernoulli_csr(shape[0], shape[1], 0.4, seed=100 + i)
        rng = np.random.default_rng(500 + i)
        data = np.array([1.5], dtype=dt) if homo else rng.standard_normal(indices.shape[0]).astype(dt)
        events = rng.random(shape[0]) < 0.1
        ev["data_%d" % i], ev["indices_%d" % i], ev["indptr_%d" % i] = data, indices, indptr
        ev["events_%d" % i], ev["shape_%d" % i] = events, np.array(shape)
        ev["out_%d" % i] = ref.csr_event_sum(data, indices, indptr, events, shape=shape)
        i += 1
  np.savez_compressed(os.path.join(HERE, "event_sum_cpu_reference.npz"), **ev)
  print("wrote", len(seq) // 3, "jitconn cases and", i, "event_sum cases")


if __name__ == "__main__":
  main()
