"""GPU parity of the jitconn operators through the C ABI.

Generator contract: stream i is std::mt19937{seed + i}; output row i of a row-walk target
(input column i of an *_atomic_* target) is what the reference's CPU kernel computes for that
single stream.  Checked against (a) golden vectors produced by the reference's compiled CPU
kernels one stream at a time, (b) the per-stream oracle, (c) exact integer probes that pin the
generated index sets, (d) full-size properties."""
import json
import os

import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
from brainpylib_amd import _lib
import benchdata as synth
from util import JIT_SHAPES, assert_close, assert_close_reordered

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
KINDS_BUILT = ("homo", "uniform", "normal")


def kernel_call(inp, *, w_kind, w_a=0.0, w_b=0.0, log_p, seed, n_row, n_col, col_walk, dense, out_dtype=None,
                device="cuda:0"):
  """Calls the custom-call target directly (homo returns counts / plain sums)."""
  t = torch.from_numpy(np.ascontiguousarray(inp)).to(device)
  if t.dtype == torch.bool:
    odt = torch.float32 if out_dtype in (None, np.float32, "float32") else torch.float64
    suffix = ("_float" if odt == torch.float32 else "_double") + "_bool"
    prefix = "gpu_event_matvec"
  else:
    odt = t.dtype
    tn = "_float" if odt == torch.float32 else "_double"
    prefix, suffix = ("gpu_matvec", tn) if dense else ("gpu_event_matvec", tn + tn)
  if w_kind == "homo":
    opaque = _lib.build_jitconn_prob_homo_descriptor(n_row, n_col, seed, log_p)
  elif w_kind == "uniform":
    # descriptor carries (w_min, w_range); the range is formed in the result type like the CPU path's b - a
    np_dt = np.float32 if odt == torch.float32 else np.float64
    opaque = _lib.build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, log_p, float(np_dt(w_a)),
                                                        float(np_dt(np_dt(w_b) - np_dt(w_a))))
  else:
    opaque = _lib.build_jitconn_prob_normal_descriptor(n_row, n_col, seed, log_p, w_a, w_b)
  out = torch.full((n_row,), 123.0, dtype=odt, device=device)  # poisoned: every element must be written
  name = prefix + ("_atomic" if col_walk else "") + "_prob_" + w_kind + "_v2" + suffix
  _lib.custom_call(name, [t, out], opaque)
  return out.cpu().numpy()


def _golden_cases():
  z = np.load(os.path.join(GOLD, "jitconn_cpu_reference.npz"))
  zs = np.load(os.path.join(GOLD, "jitconn_cpu_reference_streams.npz"))
  n = sum(1 for k in z.files if k.startswith("meta_"))
  for i in range(n):
    yield i, z["in_%d" % i], json.loads(str(z["meta_%d" % i])), zs["out_%d" % i]


def _abs_bound(oracle, inp, meta, dtype):
  """sum of |addends| per output element, for the reordering tolerance: rebuilt from the
  oracle's per-stream (index, weight) lists"""
  mag_in = np.abs(inp.astype(np.float64)) if meta["dense"] else (inp != 0).astype(np.float64)
  lp = oracle.log_p_of(meta["conn_prob"])
  n_outer, n_inner = (meta["n_col"], meta["n_row"]) if meta["col_walk"] else (meta["n_row"], meta["n_col"])
  bound = np.zeros(meta["n_row"])
  for s_ in range(n_outer):
    idx, w = oracle.jitconn_stream_weights(meta["seed"] + s_, meta["w_kind"], meta["w_a"], meta["w_b"], lp, n_inner,
                                           dtype=dtype)
    if meta["col_walk"]:
      np.add.at(bound, idx, np.abs(w.astype(np.float64)) * mag_in[s_])
    else:
      bound[s_] = (np.abs(w.astype(np.float64)) * mag_in[idx]).sum()
  return bound


def test_reference_golden_streams(cuda, oracle_mod):
  n = 0
  for i, inp, meta, want in _golden_cases():
    if meta["w_kind"] not in KINDS_BUILT:
      continue
    got = kernel_call(inp, w_kind=meta["w_kind"], w_a=meta["w_a"], w_b=meta["w_b"],
                      log_p=oracle_mod.log_p_of(meta["conn_prob"]), seed=meta["seed"], n_row=meta["n_row"],
                      n_col=meta["n_col"], col_walk=meta["col_walk"], dense=meta["dense"], out_dtype=meta["out_dtype"])
    if meta["w_kind"] == "homo" and not meta["dense"]:
      assert np.array_equal(got.astype(np.float64), want.astype(np.float64)), (i, meta)  # counts: exact
    else:
      dt = np.float32 if got.dtype == np.float32 else np.float64
      assert_close_reordered(got, want, _abs_bound(oracle_mod, inp, meta, dt), dt, what=str(meta))
    n += 1
  assert n == 450


@pytest.mark.parametrize("shape", JIT_SHAPES + [(64, 64), (3, 70000)])
@pytest.mark.parametrize("p", [0.01, 0.1, 0.5])
def test_index_sets_bit_exact_via_integer_probes(cuda, oracle_mod, shape, p):
  # dense float64 vectors 1, c and c^2 give count, sum and sum of squares of every row's index set,
  # all exact integers below 2^53: equal to the oracle's bit for bit
  n_row, n_col = shape
  lp = oracle_mod.log_p_of(p)
  c = np.arange(n_col, dtype=np.float64)
  print("case", shape, p, flush=True)
  for col_walk in (False, True):
    for vec in (np.ones(n_col), c, c * c):
      want = oracle_mod.jitconn_matvec(vec, log_p=lp, seed=1234, n_row=n_row, n_col=n_col, col_walk=col_walk,
                                       dense=True, per_stream_seed=True)
      got = kernel_call(vec, w_kind="homo", log_p=lp, seed=1234, n_row=n_row, n_col=n_col, col_walk=col_walk,
                        dense=True)
      assert np.array_equal(got, want), (shape, p, col_walk)


@pytest.mark.parametrize("n_out,n_in,p", [(3000, 1500, 0.05), (5000, 4000, 0.05), (9000, 40_000, 0.02),
                                          (20_000, 30_000, 0.03)])
def test_event_column_walk_in_every_regime(cuda, oracle_mod, n_out, n_in, p):
  # few input columns: every wave lists and seeds its own; from 2,048 columns on: a device list of the active
  # columns and generators seeded ahead, the pairs added with atomics; from ten million possible pairs on:
  # through bins.  Unit weight: the outputs are synapse counts, equal to the oracle's bit for bit, at little
  # and at much activity, twice in a row (the list's counter must be back at zero).
  lp = oracle_mod.log_p_of(p)
  rng = np.random.default_rng(n_in)
  for rate in (0.004, 0.3):
    ev = rng.random(n_in) < rate
    want = oracle_mod.jitconn_matvec(ev, log_p=lp, seed=99, n_row=n_out, n_col=n_in, col_walk=True, dense=False,
                                     per_stream_seed=True)
    for _ in range(2):
      got = kernel_call(ev, w_kind="homo", log_p=lp, seed=99, n_row=n_out, n_col=n_in, col_walk=True, dense=False)
      assert np.array_equal(got, want), (n_out, n_in, p, rate)
  # uniform weights and float events: sums of a few terms in any order
  evf = (rng.random(n_in) < 0.05).astype(np.float32)
  want = oracle_mod.jitconn_matvec(evf, log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True, dense=False,
                                   per_stream_seed=True, w_kind="uniform", w_a=-1.0, w_b=2.0)
  got = kernel_call(evf, w_kind="uniform", w_a=-1.0, w_b=2.0, log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True,
                    dense=False)
  np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("n_in", [320_000, 1_500_000, 5_000_000])
def test_row_walk_with_a_two_level_event_bitmap(cuda, oracle_mod, n_in):
  # more inputs than the 38 KB of LDS the row walk gives to a bitmap cover (311,296): a coarse
  # bitmap in LDS (one bit per 2, 8 and 32 inputs here) and the exact one in global memory, whose
  # word is looked at one batch late.  Bool and float events, all weight kinds; counts exact.
  n_out = 300
  rng = np.random.default_rng(n_in)
  ev = rng.random(n_in) < 0.02
  lp = oracle_mod.log_p_of(2000.0 / n_in)
  for inp in (ev, (ev * rng.uniform(0.5, 2.0, n_in)).astype(np.float32)):
    dense = None if inp.dtype == np.bool_ else False
    want = oracle_mod.jitconn_matvec(inp, log_p=lp, seed=77, n_row=n_out, n_col=n_in, dense=dense)
    got = kernel_call(inp, w_kind="homo", log_p=lp, seed=77, n_row=n_out, n_col=n_in, col_walk=False, dense=False)
    assert want.sum() > 0 and np.array_equal(got, want)
  for w_kind, a, b in (("uniform", 0.25, 1.75), ("normal", 0.5, 2.0)):
    want, mag = oracle_mod.jitconn_matvec(ev, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=77, n_row=n_out, n_col=n_in,
                                          return_abs=True)
    got = kernel_call(ev, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=77, n_row=n_out, n_col=n_in, col_walk=False,
                      dense=False)
    assert_close_reordered(got, want, mag, np.float32, what="two-level row walk %s" % w_kind)


def test_row_walk_lanes_past_the_end_of_a_row_count_nothing(cuda, oracle_mod):
  # two-level bitmap with EVERY event set (all coarse and exact bits are ones): the lanes of a row's last
  # batch that lie past the end of the row index words beyond the coarse bitmap, or any word of it if their
  # position wrapped; they extract a bit field of width 0 from it, so a row's count is its stream's
  # synapse count exactly.  Rows of about 3 synapses: nearly every lane of every row's only batch is past the end.
  # (8,200 outputs: the walk that seeds its generators itself)
  for n_out, n_in in ((400, 311_297), (400, 320_000), (400, 1_310_720), (8_200, 320_000)):
    ev = np.ones(n_in, dtype=np.bool_)
    lp = oracle_mod.log_p_of(3.0 / n_in)
    got = kernel_call(ev, w_kind="homo", log_p=lp, seed=123, n_row=n_out, n_col=n_in, col_walk=False, dense=False)
    want = np.array([oracle_mod.jitconn_stream_indices(123 + r, lp, n_in)[1] for r in range(n_out)], dtype=np.float32)
    assert want.sum() > 0 and np.array_equal(got, want), n_in


def test_full_matrix_recovered_by_one_hot_events(cuda, oracle_mod):
  # every entry of a 100 x 200 implicit matrix, both walks, against the per-stream oracle's index lists
  n_row, n_col, seed = 100, 200, 77
  lp = oracle_mod.log_p_of(0.1)
  M = np.zeros((n_row, n_col))
  for r in range(n_row):
    idx, _ = oracle_mod.jitconn_stream_indices(seed + r, lp, n_col)
    M[r, idx] = 1
  got = np.zeros((n_row, n_col))
  for c in range(n_col):
    ev = np.zeros(n_col, dtype=bool)
    ev[c] = True
    got[:, c] = kernel_call(ev, w_kind="homo", log_p=lp, seed=seed, n_row=n_row, n_col=n_col, col_walk=False,
                            dense=False)
  assert np.array_equal(got, M)
  # column walk of the swapped shape generates the transpose of the same matrix
  gotT = np.zeros((n_col, n_row))
  for r in range(n_row):
    ev = np.zeros(n_row, dtype=bool)
    ev[r] = True
    gotT[:, r] = kernel_call(ev, w_kind="homo", log_p=lp, seed=seed, n_row=n_col, n_col=n_row, col_walk=True,
                             dense=False)
  assert np.array_equal(gotT, M.T)
  assert M[:, 0].sum() == 0  # index 0 is never connected


def test_closed_form_and_edges(cuda, oracle_mod):
  lp = oracle_mod.log_p_of(1.0)  # every skip is 1: indices 1..n-1
  v = np.arange(1, 301, dtype=np.float64)
  out = kernel_call(v, w_kind="homo", log_p=lp, seed=3, n_row=70, n_col=300, col_walk=False, dense=True)
  assert np.array_equal(out, np.full(70, v[1:].sum()))
  out = kernel_call(v[:70].copy(), w_kind="homo", log_p=lp, seed=3, n_row=300, n_col=70, col_walk=True, dense=True)
  want = np.full(300, v[:70].sum())
  want[0] = 0
  assert np.array_equal(out, want)
  # seed + stream wraps modulo 2^32
  ev = np.random.default_rng(0).random(500) < 0.5
  lp = oracle_mod.log_p_of(0.05)
  want = oracle_mod.jitconn_matvec(ev, log_p=lp, seed=2 ** 32 - 3, n_row=10, n_col=500, per_stream_seed=True)
  got = kernel_call(ev, w_kind="homo", log_p=lp, seed=2 ** 32 - 3, n_row=10, n_col=500, col_walk=False, dense=False)
  assert np.array_equal(got, want)
  # silent input, single element, and an invalid log_p that must be refused, not looped on
  got = kernel_call(np.zeros(500, bool), w_kind="homo", log_p=lp, seed=1, n_row=10, n_col=500, col_walk=True, dense=False)
  assert not got.any()
  got = kernel_call(np.ones(1, bool), w_kind="homo", log_p=lp, seed=1, n_row=5, n_col=1, col_walk=False, dense=False)
  assert not got.any()
  with pytest.raises(RuntimeError, match="log_p must be finite and negative"):
    kernel_call(ev, w_kind="homo", log_p=0.0, seed=1, n_row=10, n_col=500, col_walk=False, dense=False)


@pytest.mark.parametrize("shape", JIT_SHAPES)
@pytest.mark.parametrize("outdim_parallel", [True, False])
def test_wrapper_determinism_and_shape_swap(cuda, shape, outdim_parallel):
  # brainpylib/_src/jitconn_ops/tests/test_event_matvec.py:63-87
  rng = np.random.default_rng(1)
  for transpose in (False, True):
    ev = rng.random(shape[0] if transpose else shape[1]) < 0.1
    kw = dict(conn_prob=0.1, seed=1234, outdim_parallel=outdim_parallel)
    r1 = bpl.event_matvec_prob_conn_homo_weight(ev, 1.5, shape=shape, transpose=transpose, **kw)
    r2 = bpl.event_matvec_prob_conn_homo_weight(ev, 1.5, shape=shape, transpose=transpose, **kw)
    r3 = bpl.event_matvec_prob_conn_homo_weight(ev, 1.5, shape=shape[::-1], transpose=not transpose, **kw)
    assert torch.equal(r1, r2) and torch.equal(r1, r3)
    assert r1.shape[0] == (shape[1] if transpose else shape[0]) and r1.dtype == torch.float32
    u1 = bpl.event_matvec_prob_conn_uniform_weight(ev, w_low=-1.0, w_high=1.0, shape=shape, transpose=transpose, **kw)
    u3 = bpl.event_matvec_prob_conn_uniform_weight(ev, w_low=-1.0, w_high=1.0, shape=shape[::-1],
                                                   transpose=not transpose, **kw)
    assert torch.allclose(u1, u3, rtol=1e-5, atol=1e-6)
    fv = rng.standard_normal(ev.shape[0]).astype(np.float32)
    m1 = bpl.matvec_prob_conn_homo_weight(fv, 0.5, shape=shape, transpose=transpose, **kw)
    m3 = bpl.matvec_prob_conn_homo_weight(fv, 0.5, shape=shape[::-1], transpose=not transpose, **kw)
    assert torch.allclose(m1, m3, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("uniform", -1.0, 1.0), ("normal", 0.5, 2.0)])
def test_row_walk_and_column_walk_are_adjoint(cuda, oracle_mod, w_kind, a, b):
  # flipping transpose AND outdim_parallel gives M^T of the same M: <y, M x> == <M^T y, x>
  n_out, n_in = 300, 500
  rng = np.random.default_rng(5)
  x = rng.integers(-3, 4, n_in).astype(np.float64)
  y = rng.integers(-3, 4, n_out).astype(np.float64)
  lp = oracle_mod.log_p_of(0.2)
  Mx = kernel_call(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=11, n_row=n_out, n_col=n_in, col_walk=False, dense=True)
  MTy = kernel_call(y, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=11, n_row=n_in, n_col=n_out, col_walk=True, dense=True)
  assert abs(y @ Mx - MTy @ x) <= 1e-9 * max(1.0, abs(y @ Mx))


@pytest.mark.parametrize("w_kind,a,b", [("uniform", 0.25, 1.75), ("normal", 0.5, 2.0)])
def test_single_weights_against_oracle_streams(cuda, oracle_mod, w_kind, a, b):
  # one-hot dense inputs isolate single weights of a stream.  Uniform weights must equal the
  # oracle's draws bit for bit; normal weights go through logf/sqrtf (libm on the host, the
  # device's own on the GPU) and may differ in the last place.
  n_row, n_col, seed = 4, 3000, 9
  lp = oracle_mod.log_p_of(0.05)
  for dt in (np.float32, np.float64):
    for r in range(n_row):
      idx, w = oracle_mod.jitconn_stream_weights(seed + r, w_kind, a, b, lp, n_col, dtype=dt)
      assert len(idx) > 100
      # all weights of the row at once: W[k] lands in output k of a column walk over one-hot ... use
      # the row walk with a one-hot per probe for a handful of positions spread over several batches
      for k in (0, 1, 2, 63, 64, 65, len(idx) // 2, len(idx) - 2, len(idx) - 1):
        e = np.zeros(n_col, dtype=dt)
        e[idx[k]] = 1
        got = kernel_call(e, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=seed, n_row=n_row, n_col=n_col,
                          col_walk=False, dense=True)
        if w_kind == "uniform":
          assert got[r] == w[k], (dt, r, k)
        else:
          assert abs(got[r] - w[k]) <= 4 * np.finfo(dt).eps * max(1.0, abs(w[k])), (dt, r, k, got[r], w[k])


def test_normal_weights_whole_rows(cuda, oracle_mod):
  # dense float64 probes c and c^2 weighted by the normal draws: compares every (index, weight)
  # pairing of long rows (many parser batches, both skip roles, batch-boundary carries)
  n_row, n_col, seed = 64, 20000, 5
  lp = oracle_mod.log_p_of(0.1)
  c = np.arange(n_col, dtype=np.float64) / n_col
  for dt in (np.float32, np.float64):
    for vec in (np.ones(n_col, dtype=dt), c.astype(dt), (c * c).astype(dt)):
      want = oracle_mod.jitconn_matvec(vec, w_kind="normal", w_a=0.1, w_b=1.0, log_p=lp, seed=seed, n_row=n_row,
                                       n_col=n_col, dense=True, per_stream_seed=True)
      got = kernel_call(vec, w_kind="normal", w_a=0.1, w_b=1.0, log_p=lp, seed=seed, n_row=n_row, n_col=n_col,
                        col_walk=False, dense=True)
      meta = dict(dense=True, conn_prob=0.1, col_walk=False, n_row=n_row, n_col=n_col, seed=seed, w_kind="normal",
                  w_a=0.1, w_b=1.0)
      assert_close_reordered(got, want, _abs_bound(oracle_mod, vec, meta, dt), dt, what="normal rows")


def test_config_jitconn_event_full_size(cuda, oracle_mod):
  # 1e6 x 1e6, conn_prob 0.001 (~1e9 implicit synapses), events 1 %, seed 42: all four flag
  # combinations.  Row walks: 300 sampled rows against single-stream oracle calls.  Column walks:
  # the whole output against the oracle run over the ~1e4 active columns only.  Plus the adjoint
  # identity between the two walks on exact integer data.
  c = synth.config_jitconn_event()
  n = c["shape"][0]
  ev = c["events"]
  lp = oracle_mod.log_p_of(c["conn_prob"])
  seed = c["seed"]
  got_row = kernel_call(ev, w_kind="homo", log_p=lp, seed=seed, n_row=n, n_col=n, col_walk=False, dense=False)
  rows = np.random.default_rng(0).choice(n, 300, replace=False)
  for r in rows:
    idx, cnt = oracle_mod.jitconn_stream_indices(seed + int(r), lp, n)
    assert cnt == idx.shape[0]
    assert got_row[r] == ev[idx].sum(), r
  got_col = kernel_call(ev, w_kind="homo", log_p=lp, seed=seed, n_row=n, n_col=n, col_walk=True, dense=False)
  want_col = np.zeros(n)
  for col in np.flatnonzero(ev):
    idx, _ = oracle_mod.jitconn_stream_indices(seed + int(col), lp, n)
    np.add.at(want_col, idx, 1.0)
  assert np.array_equal(got_col.astype(np.float64), want_col)
  # the public wrappers: weight applied afterwards, transpose only swaps the (square) shape
  w = bpl.event_matvec_prob_conn_homo_weight(ev, c["weight"], conn_prob=c["conn_prob"], shape=c["shape"], seed=seed)
  assert np.array_equal(w.cpu().numpy(), got_row * np.float32(0.1))
  wt = bpl.event_matvec_prob_conn_homo_weight(ev, c["weight"], conn_prob=c["conn_prob"], shape=c["shape"], seed=seed,
                                              transpose=True, outdim_parallel=False)
  assert np.array_equal(wt.cpu().numpy(), got_col * np.float32(0.1))
  # adjoint: <y, M x> == <M^T y, x>, counts are exact in fp32 below 2^24
  y = np.random.default_rng(1).random(n) < 0.01
  MTy = kernel_call(y, w_kind="homo", log_p=lp, seed=seed, n_row=n, n_col=n, col_walk=True, dense=False)
  assert float(got_row.astype(np.float64) @ y) == float(MTy.astype(np.float64) @ ev)


@pytest.mark.parametrize("m", [1, 5, 8, 15, 33, 64, 70, 128, 130, 300, 600, 2048])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_matmat_against_oracle_and_vmapped_matvec(cuda, oracle_mod, m, dtype):
  # m values of the reference test (matmat_testcase.py:39-44) plus tile boundaries of the kernel and row counts
  # that take several passes of 128 rows (the last one partly filled)
  k, n, seed, p = 230, 150, 7, 0.2
  X = np.random.default_rng(m).standard_normal((m, k)).astype(dtype)
  lp = oracle_mod.log_p_of(p)
  print("case", m, dtype.__name__, flush=True)
  # uniform weights: same operations in the same order as the CPU loop -> bit-exact
  want = oracle_mod.jitconn_matmat(X, w_kind="uniform", w_a=-0.5, w_b=1.5, log_p=lp, seed=seed, n=n)
  got = bpl.matmat_prob_conn_uniform_weight(X, w_low=-0.5, w_high=1.5, conn_prob=p, shape=(k, n), seed=seed).cpu().numpy()
  assert got.shape == (m, n) and np.array_equal(got, want)
  # normal weights: logf/sqrtf of the device vs libm may differ in the last place
  want, mag = oracle_mod.jitconn_matmat(X, w_kind="normal", w_a=0.0, w_b=0.01, log_p=lp, seed=seed, n=n, return_abs=True)
  got_t = bpl.matmat_prob_conn_normal_weight(X, w_mu=0.0, w_sigma=0.01, conn_prob=p, shape=(k, n), seed=seed)
  got = got_t.cpu().numpy()
  assert_close_reordered(got, want, mag, dtype, what="matmat normal")
  # the reference tests' identity: matmat(X) == vmap(matvec(transpose=True))(X)
  for i in range(0, m, max(1, m // 4)):
    yi = bpl.matvec_prob_conn_normal_weight(X[i], w_mu=0.0, w_sigma=0.01, conn_prob=p, shape=(k, n), seed=seed,
                                            transpose=True)
    assert torch.allclose(got_t[i], yi, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n", [32_768, 140_000])
def test_matmat_with_generators_seeded_ahead(cuda, oracle_mod, n):
  # from 32,768 columns of M on their generators are seeded ahead by a kernel of its own, 131,072 at a time
  # (140,000: two chunks, the second one short); uniform weights are bit-exact as with any other size
  m, k, seed, p = 9, 60, 11, 0.1
  X = np.random.default_rng(n).standard_normal((m, k)).astype(np.float32)
  lp = oracle_mod.log_p_of(p)
  want = oracle_mod.jitconn_matmat(X, w_kind="uniform", w_a=-0.5, w_b=1.5, log_p=lp, seed=seed, n=n)
  for _ in range(2):
    got = bpl.matmat_prob_conn_uniform_weight(X, w_low=-0.5, w_high=1.5, conn_prob=p, shape=(k, n), seed=seed).cpu().numpy()
    assert got.shape == (m, n) and np.array_equal(got, want)


def test_config_jitconn_matmat_full_size(cuda, oracle_mod):
  # 10,000 x 10,000 implicit matrix, conn_prob 0.1, N(0, 0.01^2) from seed 7, times B[10000, 128]:
  # out = (B^T @ M)^T in the reference's orientation (X = B^T, m = 128).
  c = synth.config_jitconn_matmat()
  X = np.ascontiguousarray(c["B"].T)
  oracle_mod.set_threads(min(16, len(os.sched_getaffinity(0))))
  lp = oracle_mod.log_p_of(c["conn_prob"])
  # the oracle on all 128 rows (every stream generated once and applied to every row of X), with
  # sum(|w x|) per output: the reordering term of the tolerance is computed, not estimated
  want, mag = oracle_mod.jitconn_matmat(X, w_kind="normal", w_a=c["w_mu"], w_b=c["w_sigma"], log_p=lp, seed=c["seed"],
                                        n=c["shape"][1], return_abs=True)
  # the definition itself (one matvec per row of X) on two rows
  rows = np.array([0, 127])
  by_rows = oracle_mod.jitconn_matmat(X[rows], w_kind="normal", w_a=c["w_mu"], w_b=c["w_sigma"], log_p=lp,
                                      seed=c["seed"], n=c["shape"][1], by_rows=True)
  oracle_mod.set_threads(1)
  assert np.array_equal(by_rows, want[rows])
  got = bpl.matmat_prob_conn_normal_weight(X, w_mu=c["w_mu"], w_sigma=c["w_sigma"], conn_prob=c["conn_prob"],
                                           shape=c["shape"], seed=c["seed"]).cpu().numpy()
  assert got.shape == (128, 10000)
  # the kernel adds in the oracle's order; what differs is the device's logf / sqrtf in the normal
  # weights (within 4 ulp each): 4 eps sum(|w x|) covers that too
  outside = assert_close_reordered(got, want, mag, np.float32, what="matmat 10,000 x 10,000 x 128")
  print("matmat full size: %d of %d outside plain rel 1e-5 / abs 1e-6; max abs err %.3e"
        % (outside, got.size, float(np.abs(got - want).max())), flush=True)


@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("uniform", 0.25, 1.75), ("normal", 0.5, 2.0)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_column_walk_through_bins_dense(cuda, oracle_mod, w_kind, a, b, dtype):
  # dense input, output wider than one 16,384-element window, > 2^20 pairs: the column walk appends
  # its pairs to bins that a second kernel adds.  Against the oracle's column walk (integer input:
  # homogeneous sums are exact) and against the row walk of the transposed flags (adjoint).
  n_out, n_in = 40_000, 2_500
  lp = oracle_mod.log_p_of(0.05)
  rng = np.random.default_rng(8)
  x = rng.integers(-3, 4, n_in).astype(dtype)
  got = kernel_call(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=21, n_row=n_out, n_col=n_in, col_walk=True,
                    dense=True)
  want, mag = oracle_mod.jitconn_matvec(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=21, n_row=n_out, n_col=n_in,
                                        col_walk=True, dense=True, return_abs=True)
  if w_kind == "homo":
    assert np.array_equal(got, want)
  else:
    assert_close_reordered(got, want, mag, dtype, what="binned column walk %s" % w_kind)
  y = rng.integers(-3, 4, n_out).astype(np.float64)
  x64 = x.astype(np.float64)
  Mx = kernel_call(x64, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=21, n_row=n_out, n_col=n_in, col_walk=True, dense=True)
  MTy = kernel_call(y, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=21, n_row=n_in, n_col=n_out, col_walk=False, dense=True)
  assert abs(y @ Mx - MTy @ x64) <= 1e-9 * max(1.0, abs(y @ Mx))


@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("uniform", 0.25, 1.75)])
@pytest.mark.parametrize("n_out,n_in,p,dtype", [(3_000_000, 300, 0.0015, np.float32), (3_000_000, 300, 0.0015, np.float64),
                                                (9_000_000, 100, 0.0015, np.float32)])
def test_column_walk_through_bins_wide_windows(cuda, oracle_mod, w_kind, a, b, n_out, n_in, p, dtype):
  # outputs of more than two million elements: the windows grow beyond the 16,384 accumulators a workgroup
  # holds at once (3,000,000: windows of 32,768 outputs added in two slices, pairs still packed with 16-bit
  # positions; 9,000,000: windows of 131,072 outputs in eight slices, whole pairs).  Integer input: the
  # homogeneous sums are exact.
  lp = oracle_mod.log_p_of(p)
  rng = np.random.default_rng(n_out % 1000)
  x = rng.integers(-3, 4, n_in).astype(dtype)
  x[x == 0] = 1
  got = kernel_call(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True, dense=True)
  want, mag = oracle_mod.jitconn_matvec(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in,
                                        col_walk=True, dense=True, return_abs=True)
  assert mag.sum() > 1_048_576  # (enough pairs for the bins)
  if w_kind == "homo":
    assert np.array_equal(got, want)
  else:
    assert_close_reordered(got, want, mag, dtype, what="binned column walk, wide windows")


@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("normal", 0.5, 2.0)])
@pytest.mark.parametrize("n_out,n_in,p", [(4000, 4000, 0.02), (700, 90, 0.3), (5, 3, 0.9), (30_000, 2047, 0.01),
                                          (2 ** 24 + 5, 7, 2e-6), (2 ** 24 + 5, 140_000, 4e-7)])
def test_column_walk_dense_with_few_pairs(cuda, oracle_mod, w_kind, a, b, n_out, n_in, p):
  # dense input and fewer than 2^20 possible pairs: every column's generator is seeded ahead and the walk adds
  # its pairs to the output with atomics (no bins).  Against the oracle's column walk; integer input, so the
  # homogeneous sums are exact.  And a bound on the time: with every lane seeding its own column's generator
  # the first shape took 0.5 ms.
  lp = oracle_mod.log_p_of(p)
  x = np.random.default_rng(n_in).integers(-3, 4, n_in).astype(np.float32)
  kw = dict(w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=33, n_row=n_out, n_col=n_in, col_walk=True, dense=True)
  got = kernel_call(x, **kw)
  want, mag = oracle_mod.jitconn_matvec(x, return_abs=True, **kw)
  if w_kind == "homo":
    assert np.array_equal(got, want)
  else:
    assert_close_reordered(got, want, mag, np.float32, what="dense column walk with few pairs")
  if n_out == 4000 and w_kind == "homo":
    xd = torch.from_numpy(x).cuda()
    call = lambda: bpl.matvec_prob_conn_homo_weight(xd, 0.5, conn_prob=p, shape=(n_out, n_in), seed=33, outdim_parallel=False)
    call()
    torch.cuda.synchronize()
    # best of five groups of five calls (a shared box or low clocks slow single groups down): about 70 us when the
    # generators are seeded ahead, 500 us when every lane seeds its own
    best = float("inf")
    for _ in range(5):
      e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
      e0.record()
      for _ in range(5):
        call()
      e1.record()
      torch.cuda.synchronize()
      best = min(best, e0.elapsed_time(e1) * 1e3 / 5)
    print("dense column walk 4,000 x 4,000: %.1f us per call (best of 5 groups)" % best, flush=True)
    assert best < 300.0


def test_column_walk_through_bins_sliced_windows(cuda, oracle_mod):
  # more than 2^21 outputs: the bins' windows are wider than their accumulators in LDS and are
  # added in slices
  n_out, n_in = 3_000_001, 1_500
  lp = oracle_mod.log_p_of(0.0004)
  rng = np.random.default_rng(9)
  x = rng.integers(-3, 4, n_in).astype(np.float32)
  for w_kind, a, b in (("homo", 0.0, 0.0), ("uniform", 0.25, 1.75)):
    got = kernel_call(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True, dense=True)
    want, mag = oracle_mod.jitconn_matvec(x, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in,
                                          col_walk=True, dense=True, return_abs=True)
    if w_kind == "homo":
      assert np.array_equal(got, want)
    else:
      assert_close_reordered(got, want, mag, np.float32, what="sliced binned column walk")


def test_column_walk_through_bins_events_and_overflow(cuda, oracle_mod):
  # event input with n_in * n_out * p >= 5e7: bins sized for one active column in eight.  At 2 % activity
  # everything fits; with every column active most pairs overflow into direct atomics.  Counts are exact.
  n_out, n_in = 60_000, 90_000
  lp = oracle_mod.log_p_of(0.01)
  rng = np.random.default_rng(9)
  for rate in (0.02, 1.0):
    ev = rng.random(n_in) < rate
    print("rate", rate, flush=True)
    got = kernel_call(ev, w_kind="homo", log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True, dense=False)
    want = oracle_mod.jitconn_matvec(ev, w_kind="homo", log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=True)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_walks_weights_and_inputs_against_oracle(cuda, oracle_mod, seed):
  # shapes up to two million inputs / outputs, both walks, all weight kinds, bool / float events and
  # dense vectors drawn at random: every target of the family against the oracle
  rng = np.random.default_rng(seed)
  for case in range(100):
    n_out = int(10 ** rng.uniform(0, 4.0))
    n_in = int(10 ** rng.uniform(0, 6.3))
    col_walk = bool(rng.random() < 0.5)
    if col_walk:
      n_out, n_in = int(10 ** rng.uniform(0, 6.3)), int(10 ** rng.uniform(0, 3.7))
    syn = 10 ** rng.uniform(0, 2.5)
    p = min(1.0, syn / max(n_out if col_walk else n_in, 1))
    lp = oracle_mod.log_p_of(p)
    w_kind = str(rng.choice(["homo", "uniform", "normal"]))
    a, b = (0.0, 0.0) if w_kind == "homo" else (0.25, 1.75)
    dtype = np.float32 if rng.random() < 0.7 else np.float64
    kind = str(rng.choice(["bool", "float", "dense"]))
    if kind == "bool":
      inp, dense = rng.random(n_in) < rng.choice([0.0, 0.02, 0.5, 1.0]), False
    elif kind == "float":
      inp, dense = ((rng.random(n_in) < 0.3) * rng.uniform(0.5, 2, n_in)).astype(dtype), False
    else:
      inp, dense = rng.integers(-3, 4, n_in).astype(dtype), True
    stream_seed = int(rng.integers(0, 2 ** 31))
    print("case", case, n_out, n_in, col_walk, "%.2e" % p, w_kind, kind, dtype.__name__, flush=True)
    want, mag = oracle_mod.jitconn_matvec(inp, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=stream_seed, n_row=n_out,
                                          n_col=n_in, col_walk=col_walk, dense=(None if kind == "bool" else dense),
                                          return_abs=True)
    got = kernel_call(inp, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=stream_seed, n_row=n_out, n_col=n_in,
                      col_walk=col_walk, dense=dense)
    if w_kind == "homo":
      assert np.array_equal(got, want)  # counts / sums of small integers
    else:
      assert_close_reordered(got, want, mag, np.float32 if kind == "bool" else dtype, what="case %d" % case)



@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("uniform", 0.25, 1.75), ("normal", 0.5, 2.0)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_first_generation_dense_targets_give_the_cpu_paths_matrix(cuda, oracle_mod, w_kind, a, b, dtype):
  # gpu_matvec_prob_*_v1_*: the descriptor carries conn_prob itself; on the reference's CPU path the
  # version does not change the result (matvec.py:296-308), so the oracle is the same row walk.
  n_row, n_col, seed = 70, 3000, 21
  rng = np.random.default_rng(3)
  tn = "_float" if dtype == np.float32 else "_double"
  np_dt = dtype
  for p, vec in ((0.07, rng.integers(-3, 4, n_col).astype(dtype)), (0.5, np.arange(n_col).astype(dtype)),
                 (1.0, np.ones(n_col, dtype=dtype))):
    lp = oracle_mod.log_p_of(p)
    want = oracle_mod.jitconn_matvec(vec, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=seed, n_row=n_row, n_col=n_col,
                                     dense=True, per_stream_seed=True)
    if w_kind == "homo":
      opaque = _lib.build_jitconn_prob_homo_descriptor(n_row, n_col, seed, p)
    elif w_kind == "uniform":
      opaque = _lib.build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, p, float(np_dt(a)),
                                                          float(np_dt(np_dt(b) - np_dt(a))))
    else:
      opaque = _lib.build_jitconn_prob_normal_descriptor(n_row, n_col, seed, p, a, b)
    t = torch.from_numpy(vec).to("cuda:0")
    out = torch.full((n_row,), 123.0, dtype=t.dtype, device="cuda:0")
    _lib.custom_call("gpu_matvec_prob_" + w_kind + "_v1" + tn, [t, out], opaque)
    got = out.cpu().numpy()
    v2 = kernel_call(vec, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=seed, n_row=n_row, n_col=n_col, col_walk=False,
                     dense=True)
    assert np.array_equal(got, v2), (w_kind, p)  # one kernel behind both names
    if w_kind == "homo":
      assert np.array_equal(got.astype(np.float64), want.astype(np.float64)), p  # integer data: exact sums
      if p >= 1.0:
        assert np.all(got == n_col - 1)  # closed form: every index from 1 on
    else:
      meta = dict(dense=True, conn_prob=p, col_walk=False, n_row=n_row, n_col=n_col, seed=seed, w_kind=w_kind,
                  w_a=a, w_b=b)
      assert_close_reordered(got, want, _abs_bound(oracle_mod, vec, meta, dtype), dtype, what="v1 " + w_kind)


def test_version_argument_of_the_dense_wrappers(cuda):
  rng = np.random.default_rng(8)
  shape = (200, 300)
  kw = dict(conn_prob=0.1, shape=shape, seed=77)
  for transpose in (False, True):
    v = rng.standard_normal(shape[0] if transpose else shape[1]).astype(np.float32)
    calls = ((bpl.matvec_prob_conn_homo_weight, (v, 0.3), {}),
             (bpl.matvec_prob_conn_uniform_weight, (v,), dict(w_low=-1.0, w_high=2.0)),
             (bpl.matvec_prob_conn_normal_weight, (v,), dict(w_mu=0.1, w_sigma=0.5)))
    for fn, args, extra in calls:
      y1 = fn(*args, transpose=transpose, version='v1', **extra, **kw)
      y2 = fn(*args, transpose=transpose, version='v2', **extra, **kw)
      assert torch.equal(y1, y2), fn.__name__
      with pytest.raises(_lib.GPUOperatorNotFound):  # the reference registers no atomic v1 target either
        fn(*args, transpose=transpose, outdim_parallel=False, version='v1', **extra, **kw)
      with pytest.raises(AssertionError):
        fn(*args, transpose=transpose, version='v3', **extra, **kw)
  # the raw probability is validated where it is converted
  t = torch.zeros(10, dtype=torch.float32, device="cuda:0")
  out = torch.zeros(10, dtype=torch.float32, device="cuda:0")
  with pytest.raises(RuntimeError):
    _lib.custom_call("gpu_matvec_prob_homo_v1_float", [t, out], _lib.build_jitconn_prob_homo_descriptor(10, 10, 1, -0.5))


@pytest.mark.parametrize("n_out,n_in", [(8192, 3000), (10_007, 200_000), (20_000, 400_000), (70_001, 5000)])
def test_row_walk_with_generators_seeded_inside_the_kernel(cuda, oracle_mod, n_out, n_in):
  # from 8,192 outputs the row walk seeds its generators itself, 64 streams at a time, into rings of
  # seeded states that its workgroups keep in device memory: whole outputs against the per-stream
  # oracle for every weight kind, event (LDS bitmap / two-level bitmap / packed float events) and
  # dense input, output counts that are and are not multiples of 64, fewer batches than workgroups,
  # twice in a row (the second call finds the rings of the first).
  rng = np.random.default_rng(n_out)
  lp = oracle_mod.log_p_of(200.0 / n_in)
  ev = rng.random(n_in) < 0.1
  fev = (ev * rng.uniform(0.5, 2.0, n_in)).astype(np.float32)
  vec = rng.integers(-3, 4, n_in).astype(np.float64)
  print("case", n_out, n_in, flush=True)
  for _ in range(2):
    for inp, dense in ((ev, False), (fev, False), (vec, True)):
      want = oracle_mod.jitconn_matvec(inp, log_p=lp, seed=5, n_row=n_out, n_col=n_in, dense=dense, per_stream_seed=True)
      got = kernel_call(inp, w_kind="homo", log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=False, dense=dense)
      assert want.any() and np.array_equal(got.astype(np.float64), want.astype(np.float64)), (inp.dtype, dense)
  for w_kind, a, b in (("uniform", 0.25, 1.75), ("normal", 0.5, 2.0)):
    for inp, dense, dt in ((ev, False, np.float32), (vec.astype(np.float32), True, np.float32), (vec, True, np.float64)):
      want, mag = oracle_mod.jitconn_matvec(inp, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in,
                                            dense=dense, per_stream_seed=True, return_abs=True)
      got = kernel_call(inp, w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=5, n_row=n_out, n_col=n_in, col_walk=False,
                        dense=dense)
      assert_close_reordered(got, want, mag, dt, what="fused row walk %s" % w_kind)
